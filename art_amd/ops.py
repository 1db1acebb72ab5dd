"""Tensor-level wrappers of the artk C-ABI: validate layouts, allocate outputs and
workspace with torch, pass raw pointers and the current HIP stream.

Every function here requires tensors on a ROCm device and the built HIP
library; nothing falls back to torch math.
"""
from __future__ import annotations

import weakref
from typing import Optional, Tuple

import torch

from . import _lib

DEFAULT_CHUNK_TOKENS = 0  # 0: the library picks (about 6000 positions, split evenly)
FUSED_SKIP_INACTIVE = 1   # ARTK_FUSED_SKIP_INACTIVE


def _stream(device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _need(t: torch.Tensor, name: str, dtype: torch.dtype, shape=None) -> torch.Tensor:
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name} must be a tensor")
    if not t.is_cuda:
        raise ValueError(f"{name} must live on the GPU (got {t.device}); there is no CPU path")
    if t.dtype != dtype:
        raise TypeError(f"{name} must be {dtype}, got {t.dtype}")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise ValueError(f"{name} must have shape {tuple(shape)}, got {tuple(t.shape)}")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")
    return t


def _workspace(nbytes: int, device) -> torch.Tensor:
    return torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=device)


def _mask_u8(mask: torch.Tensor) -> torch.Tensor:
    if mask.dtype == torch.bool:
        return mask.view(torch.uint8)
    if mask.dtype == torch.uint8:
        return mask
    raise TypeError(f"mask must be bool or uint8, got {mask.dtype}")


# -----------------------------------------------------------------------------
# transposed copies of frozen weights
# -----------------------------------------------------------------------------
_transpose_cache: "dict[int, tuple]" = {}
_frozen_cache: "dict[int, tuple]" = {}


def transpose(x: torch.Tensor) -> torch.Tensor:
    """out[c, r] = x[r, c] for a contiguous bf16 matrix."""
    _need(x, "x", torch.bfloat16)
    if x.dim() != 2:
        raise ValueError("x must be 2-D")
    R, C = x.shape
    out = torch.empty((C, R), dtype=torch.bfloat16, device=x.device)
    _lib.check(_lib.load().artk_transpose_bf16(x.data_ptr(), out.data_ptr(), R, C, _stream(x.device)))
    return out


def transposed_weight(w: torch.Tensor) -> torch.Tensor:
    """Transposed copy of a (frozen) weight, cached until the weight is modified
    in place or freed.  The backward GEMMs need the weight with its other
    dimension contiguous; the copy is made once per weight version."""
    key = id(w)
    hit = _transpose_cache.get(key)
    if hit is not None:
        ref, version, ptr, wt = hit
        if ref() is w and version == w._version and ptr == w.data_ptr():
            return wt
    wt = transpose(w)
    try:
        ref = weakref.ref(w, lambda _r, k=key: _transpose_cache.pop(k, None))
    except TypeError:  # pragma: no cover
        return wt
    _transpose_cache[key] = (ref, w._version, w.data_ptr(), wt)
    return wt


def frozen_bf16(w: torch.Tensor) -> torch.Tensor:
    """A detached bf16 view (or copy, if ``w`` has another dtype) of a frozen weight that is
    the *same tensor object* from call to call for as long as ``w`` is not modified in place,
    so that per-weight caches keyed by the object (``transposed_weight``) keep hitting when a
    caller starts from ``module.weight`` in every step."""
    key = id(w)
    hit = _frozen_cache.get(key)
    if hit is not None:
        ref, version, ptr, out = hit
        if ref() is w and version == w._version and ptr == w.data_ptr():
            return out
    out = w.detach()
    if out.dtype != torch.bfloat16:
        out = out.to(torch.bfloat16)
    out = out.contiguous()
    try:
        ref = weakref.ref(w, lambda _r, k=key: _frozen_cache.pop(k, None))
    except TypeError:  # pragma: no cover
        return out
    _frozen_cache[key] = (ref, w._version, w.data_ptr(), out)
    return out


def gemm_nt(p: torch.Tensor, q: torch.Tensor, out_f32: bool = False) -> torch.Tensor:
    """out[n, m] = sum_k q[n, k] * p[m, k] through the shared MFMA main loop."""
    _need(p, "p", torch.bfloat16)
    _need(q, "q", torch.bfloat16)
    M, K = p.shape
    N, K2 = q.shape
    if K != K2:
        raise ValueError("inner dimensions differ")
    out = torch.empty((N, M), dtype=torch.float32 if out_f32 else torch.bfloat16, device=p.device)
    _lib.check(
        _lib.load().artk_gemm_nt(p.data_ptr(), q.data_ptr(), out.data_ptr(), M, N, K, int(out_f32),
                                 _stream(p.device))
    )
    return out


# -----------------------------------------------------------------------------
# logprob forward / backward
# -----------------------------------------------------------------------------
def logprob_fwd(hidden: torch.Tensor, lm_head: torch.Tensor, ids: torch.Tensor, shift: bool,
                row_len: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """(logprob, lse), both f32 [T].  hidden bf16 [T,H], lm_head bf16 [V,H], ids int64 [T]."""
    T, H = hidden.shape
    V = lm_head.shape[0]
    _need(hidden, "hidden", torch.bfloat16)
    _need(lm_head, "lm_head", torch.bfloat16, (V, H))
    _need(ids, "ids", torch.int64, (T,))
    lib = _lib.load()
    dev = hidden.device
    logprob = torch.empty(T, dtype=torch.float32, device=dev)
    lse = torch.empty(T, dtype=torch.float32, device=dev)
    ws = _workspace(lib.artk_logprob_fwd_workspace_bytes(T, V, H), dev)
    _lib.check(
        lib.artk_logprob_fwd(hidden.data_ptr(), lm_head.data_ptr(), ids.data_ptr(), int(shift), T,
                             row_len, V, H, logprob.data_ptr(), lse.data_ptr(), ws.data_ptr(),
                             ws.numel(), _stream(dev))
    )
    return logprob, lse


def logprob_bwd(hidden, lm_head, lm_head_t, ids, shift: bool, row_len: int, lse, grad_logprob,
                chunk_tokens: int = DEFAULT_CHUNK_TOKENS) -> torch.Tensor:
    """d_hidden bf16 [T,H] for upstream gradient grad_logprob f32 [T]."""
    T, H = hidden.shape
    V = lm_head.shape[0]
    _need(hidden, "hidden", torch.bfloat16)
    _need(lm_head, "lm_head", torch.bfloat16, (V, H))
    _need(lm_head_t, "lm_head_t", torch.bfloat16, (H, V))
    _need(ids, "ids", torch.int64, (T,))
    _need(lse, "lse", torch.float32, (T,))
    _need(grad_logprob, "grad_logprob", torch.float32, (T,))
    lib = _lib.load()
    dev = hidden.device
    d_hidden = torch.empty((T, H), dtype=torch.bfloat16, device=dev)
    ws = _workspace(lib.artk_logprob_bwd_workspace_bytes(T, V, H, chunk_tokens), dev)
    _lib.check(
        lib.artk_logprob_bwd(hidden.data_ptr(), lm_head.data_ptr(), lm_head_t.data_ptr(),
                             ids.data_ptr(), int(shift), T, row_len, V, H, lse.data_ptr(),
                             grad_logprob.data_ptr(), d_hidden.data_ptr(), chunk_tokens,
                             ws.data_ptr(), ws.numel(), _stream(dev))
    )
    return d_hidden


# -----------------------------------------------------------------------------
# loss
# -----------------------------------------------------------------------------
def clip_bounds(epsilon: float, epsilon_high: Optional[float]) -> Tuple[float, float]:
    """1 - epsilon and 1 + epsilon_high as the reference forms them in Python
    floats (src/art/local/train.py:125-131) before torch narrows them to f32."""
    if epsilon_high is None:
        epsilon_high = epsilon
    return 1 - epsilon, 1 + epsilon_high


def grpo_loss(new_logprob, old_logprob, advantages, mask, weights, ref_logprob, shift: bool,
              row_len: int, clip_lo: float, clip_hi: float, beta: float,
              want_coef: bool = True) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """scalars f32 [4] = (loss, mean_policy_loss, mean_kl, mask_count) and
    coef f32 [T] = d loss / d new_logprob."""
    T = new_logprob.numel()
    _need(new_logprob, "new_logprob", torch.float32, (T,))
    _need(old_logprob, "old_logprob", torch.float32, (T,))
    _need(advantages, "advantages", torch.float32, (T,))
    _need(weights, "weights", torch.float32, (T,))
    mask = _need(_mask_u8(mask), "mask", torch.uint8, (T,))
    if ref_logprob is not None:
        _need(ref_logprob, "ref_logprob", torch.float32, (T,))
    lib = _lib.load()
    dev = new_logprob.device
    scalars = torch.empty(4, dtype=torch.float32, device=dev)
    coef = torch.empty(T, dtype=torch.float32, device=dev) if want_coef else None
    ws = _workspace(lib.artk_grpo_loss_workspace_bytes(T), dev)
    _lib.check(
        lib.artk_grpo_loss(new_logprob.data_ptr(), old_logprob.data_ptr(), advantages.data_ptr(),
                           mask.data_ptr(), weights.data_ptr(), _ptr(ref_logprob), int(shift), T,
                           row_len, clip_lo, clip_hi, beta, scalars.data_ptr(), _ptr(coef),
                           ws.data_ptr(), ws.numel(), _stream(dev))
    )
    return scalars, coef


def grpo_fused(hidden, lm_head, lm_head_t, tokens, old_logprob, advantages, mask, weights,
               ref_logprob, row_len: int, clip_lo: float, clip_hi: float, beta: float,
               chunk_tokens: int = DEFAULT_CHUNK_TOKENS, workspace: Optional[torch.Tensor] = None,
               out: Optional[tuple] = None, skip_inactive: bool = False):
    """One call for loss and d_hidden of a packed batch given its hidden states.

    All per-token inputs are the un-shifted PackedTensors rows flattened to [T].
    Returns (scalars f32 [5] = (loss, mean_policy_loss, mean_kl, mask_count, dropped_rows),
    logprob f32 [T], d_hidden bf16 [T,H]).  dropped_rows counts rows whose target has
    probability below e^-80 under the current policy: their d_hidden row is zero.  With
    skip_inactive the lm_head projection runs only for positions that can
    contribute to the loss; logprob is NaN elsewhere."""
    T, H = hidden.shape
    V = lm_head.shape[0]
    _need(hidden, "hidden", torch.bfloat16)
    _need(lm_head, "lm_head", torch.bfloat16, (V, H))
    _need(lm_head_t, "lm_head_t", torch.bfloat16, (H, V))
    _need(tokens, "tokens", torch.int64, (T,))
    _need(old_logprob, "old_logprob", torch.float32, (T,))
    _need(advantages, "advantages", torch.float32, (T,))
    _need(weights, "weights", torch.float32, (T,))
    mask = _need(_mask_u8(mask), "mask", torch.uint8, (T,))
    if ref_logprob is not None:
        _need(ref_logprob, "ref_logprob", torch.float32, (T,))
    lib = _lib.load()
    dev = hidden.device
    if out is None:
        scalars = torch.empty(5, dtype=torch.float32, device=dev)
        logprob = torch.empty(T, dtype=torch.float32, device=dev)
        d_hidden = torch.empty((T, H), dtype=torch.bfloat16, device=dev)
    else:
        scalars, logprob, d_hidden = out
        _need(scalars, "scalars", torch.float32, (5,))
    need = lib.artk_grpo_fused_workspace_bytes(T, V, H, chunk_tokens)
    ws = workspace if workspace is not None else _workspace(need, dev)
    _lib.check(
        lib.artk_grpo_fused(hidden.data_ptr(), lm_head.data_ptr(), lm_head_t.data_ptr(),
                            tokens.data_ptr(), old_logprob.data_ptr(), advantages.data_ptr(),
                            mask.data_ptr(), weights.data_ptr(), _ptr(ref_logprob), T, row_len, V,
                            H, clip_lo, clip_hi, beta, chunk_tokens,
                            FUSED_SKIP_INACTIVE if skip_inactive else 0, scalars.data_ptr(),
                            logprob.data_ptr(), d_hidden.data_ptr(), ws.data_ptr(), ws.numel(),
                            _stream(dev))
    )
    return scalars, logprob, d_hidden


def grpo_fused_workspace_bytes(T: int, V: int, H: int, chunk_tokens: int = DEFAULT_CHUNK_TOKENS) -> int:
    return int(_lib.load().artk_grpo_fused_workspace_bytes(T, V, H, chunk_tokens))


# -----------------------------------------------------------------------------
# LoRA linear
# -----------------------------------------------------------------------------
def lora_linear_fwd(x, W, A, B, scale: float, bias: Optional[torch.Tensor] = None):
    """(y bf16 [T,out], xa f32 [T,r]) for x bf16 [T,in], W bf16 [out,in], A bf16 [r,in], B bf16 [out,r]
    and an optional frozen bias bf16 [out] (added in the GEMM epilogue)."""
    T, n_in = x.shape
    n_out, r = B.shape
    _need(x, "x", torch.bfloat16)
    _need(W, "W", torch.bfloat16, (n_out, n_in))
    _need(A, "A", torch.bfloat16, (r, n_in))
    _need(B, "B", torch.bfloat16, (n_out, r))
    if bias is not None:
        _need(bias, "bias", torch.bfloat16, (n_out,))
    lib = _lib.load()
    dev = x.device
    y = torch.empty((T, n_out), dtype=torch.bfloat16, device=dev)
    xa = torch.empty((T, r), dtype=torch.float32, device=dev)
    ws = _workspace(lib.artk_lora_linear_fwd_workspace_bytes(T, n_in, n_out, r), dev)
    _lib.check(
        lib.artk_lora_linear_fwd(x.data_ptr(), W.data_ptr(), A.data_ptr(), B.data_ptr(), _ptr(bias), scale,
                                 T, n_in, n_out, r, y.data_ptr(), xa.data_ptr(), ws.data_ptr(),
                                 ws.numel(), _stream(dev))
    )
    return y, xa


def lora_linear_bwd(g, x, W_t, A, B, xa, scale: float):
    """(dx bf16 [T,in], dA f32 [r,in], dB f32 [out,r]) for upstream gradient g bf16 [T,out]."""
    T, n_in = x.shape
    n_out, r = B.shape
    _need(g, "g", torch.bfloat16, (T, n_out))
    _need(x, "x", torch.bfloat16)
    _need(W_t, "W_t", torch.bfloat16, (n_in, n_out))
    _need(A, "A", torch.bfloat16, (r, n_in))
    _need(B, "B", torch.bfloat16, (n_out, r))
    _need(xa, "xa", torch.float32, (T, r))
    lib = _lib.load()
    dev = x.device
    dx = torch.empty((T, n_in), dtype=torch.bfloat16, device=dev)
    dA = torch.empty((r, n_in), dtype=torch.float32, device=dev)
    dB = torch.empty((n_out, r), dtype=torch.float32, device=dev)
    ws = _workspace(lib.artk_lora_linear_bwd_workspace_bytes(T, n_in, n_out, r), dev)
    _lib.check(
        lib.artk_lora_linear_bwd(g.data_ptr(), x.data_ptr(), W_t.data_ptr(), A.data_ptr(),
                                 B.data_ptr(), xa.data_ptr(), scale, T, n_in, n_out, r, dx.data_ptr(),
                                 dA.data_ptr(), dB.data_ptr(), ws.data_ptr(), ws.numel(), _stream(dev))
    )
    return dx, dA, dB


# -----------------------------------------------------------------------------
# MoE expert path
# -----------------------------------------------------------------------------
class Routing:
    """Device tensors that describe one routing decision (see artk_moe_route)."""

    __slots__ = ("topk_idx", "topk_w", "perm", "inv_perm", "row_token", "offsets", "tile_prefix",
                 "blk_prefix", "n_rows", "n_experts", "k")


def moe_route(router_logits: torch.Tensor, k: int) -> Routing:
    T, E = router_logits.shape
    _need(router_logits, "router_logits", torch.float32)
    lib = _lib.load()
    dev = router_logits.device
    i32 = lambda *shape: torch.empty(shape, dtype=torch.int32, device=dev)
    r = Routing()
    r.topk_idx, r.topk_w = i32(T, k), torch.empty((T, k), dtype=torch.float32, device=dev)
    r.perm, r.inv_perm, r.row_token = i32(T * k), i32(T * k), i32(T * k)
    r.offsets, r.tile_prefix, r.blk_prefix = i32(E + 1), i32(E + 1), i32(E + 1)
    r.n_rows, r.n_experts, r.k = T * k, E, k
    ws = _workspace(lib.artk_moe_route_workspace_bytes(T, E, k), dev)
    _lib.check(
        lib.artk_moe_route(router_logits.data_ptr(), T, E, k, r.topk_idx.data_ptr(),
                           r.topk_w.data_ptr(), r.perm.data_ptr(), r.inv_perm.data_ptr(),
                           r.row_token.data_ptr(), r.offsets.data_ptr(), r.tile_prefix.data_ptr(),
                           r.blk_prefix.data_ptr(), ws.data_ptr(), ws.numel(), _stream(dev))
    )
    return r


def transpose_batched(x: torch.Tensor) -> torch.Tensor:
    """out[b, c, r] = x[b, r, c] for a contiguous bf16 [n, R, C] tensor."""
    _need(x, "x", torch.bfloat16)
    n, R, C = x.shape
    out = torch.empty((n, C, R), dtype=torch.bfloat16, device=x.device)
    _lib.check(_lib.load().artk_transpose_bf16_batched(x.data_ptr(), out.data_ptr(), n, R, C,
                                                        _stream(x.device)))
    return out


def moe_lora_grouped_fwd(x, gather, W, A, B, scale: float, routing: Routing):
    """(y bf16 [n_rows,out], xa f32 [n_rows,r]); x bf16 [*,in], W bf16 [E,out,in]."""
    E, n_out, n_in = W.shape
    r = A.shape[1]
    _need(x, "x", torch.bfloat16)
    _need(W, "W", torch.bfloat16)
    _need(A, "A", torch.bfloat16, (E, r, n_in))
    _need(B, "B", torch.bfloat16, (E, n_out, r))
    if gather is not None:
        _need(gather, "gather", torch.int32, (routing.n_rows,))
    elif x.shape[0] != routing.n_rows:
        raise ValueError("x must have one row per sorted (token, expert) pair when gather is None")
    lib = _lib.load()
    dev = x.device
    n = routing.n_rows
    y = torch.empty((n, n_out), dtype=torch.bfloat16, device=dev)
    xa = torch.empty((n, r), dtype=torch.float32, device=dev)
    ws = _workspace(lib.artk_moe_lora_grouped_fwd_workspace_bytes(n, n_in, n_out, E, r), dev)
    _lib.check(
        lib.artk_moe_lora_grouped_fwd(x.data_ptr(), _ptr(gather), W.data_ptr(), A.data_ptr(),
                                      B.data_ptr(), scale, routing.offsets.data_ptr(),
                                      routing.tile_prefix.data_ptr(), routing.blk_prefix.data_ptr(), n,
                                      n_in, n_out, E, r, y.data_ptr(), xa.data_ptr(), ws.data_ptr(),
                                      ws.numel(), _stream(dev))
    )
    return y, xa


def moe_lora_grouped_bwd(g, x, gather, W_t, A, B, xa, scale: float, routing: Routing):
    """(dx bf16 [n_rows,in], dA f32 [E,r,in], dB f32 [E,out,r])."""
    E, n_in, n_out = W_t.shape
    r = A.shape[1]
    n = routing.n_rows
    _need(g, "g", torch.bfloat16, (n, n_out))
    _need(x, "x", torch.bfloat16)
    _need(W_t, "W_t", torch.bfloat16)
    _need(xa, "xa", torch.float32, (n, r))
    lib = _lib.load()
    dev = x.device
    dx = torch.empty((n, n_in), dtype=torch.bfloat16, device=dev)
    dA = torch.empty((E, r, n_in), dtype=torch.float32, device=dev)
    dB = torch.empty((E, n_out, r), dtype=torch.float32, device=dev)
    ws = _workspace(lib.artk_moe_lora_grouped_bwd_workspace_bytes(n, n_in, n_out, E, r), dev)
    _lib.check(
        lib.artk_moe_lora_grouped_bwd(g.data_ptr(), x.data_ptr(), _ptr(gather), W_t.data_ptr(),
                                      A.data_ptr(), B.data_ptr(), xa.data_ptr(), scale,
                                      routing.offsets.data_ptr(), routing.tile_prefix.data_ptr(),
                                      routing.blk_prefix.data_ptr(), n, n_in, n_out, E, r,
                                      dx.data_ptr(), dA.data_ptr(), dB.data_ptr(), ws.data_ptr(),
                                      ws.numel(), _stream(dev))
    )
    return dx, dA, dB


# -----------------------------------------------------------------------------
# Packed-row attention
# -----------------------------------------------------------------------------
class AttnPlan:
    """Device-side description of one packed row's visibility (see artk_attn_plan)."""

    __slots__ = ("buf", "S")


def attn_plan(group_ids: torch.Tensor, parent_ids: torch.Tensor) -> AttnPlan:
    """Plan for one packed row: ids are the int64 [S] PackedTensors rows."""
    S = group_ids.numel()
    _need(group_ids, "group_ids", torch.int64, (S,))
    _need(parent_ids, "parent_ids", torch.int64, (S,))
    lib = _lib.load()
    dev = group_ids.device
    plan = AttnPlan()
    plan.S = S
    plan.buf = torch.empty(lib.artk_attn_plan_bytes(S), dtype=torch.uint8, device=dev)
    _lib.check(lib.artk_attn_plan(group_ids.data_ptr(), parent_ids.data_ptr(), S, plan.buf.data_ptr(),
                                  plan.buf.numel(), _stream(dev)))
    return plan


def _shd(t: torch.Tensor, name: str):
    """(stride_s, stride_h) of a bf16 [S, H, D] view whose last dimension is contiguous."""
    if t.dtype != torch.bfloat16 or t.dim() != 3 or t.stride(2) != 1 or not t.is_cuda:
        raise ValueError(f"{name}: expected a bf16 device tensor [S, H, D] with contiguous D")
    return t.stride(0), t.stride(1)


def attn_fwd(q, k, v, plan: AttnPlan, scale: Optional[float] = None):
    """(out bf16 [S, Hq, D], lse f32 [Hq, S]) for q [S, Hq, D], k/v [S, Hkv, D] (any strides over S, H)."""
    S, Hq, D = q.shape
    Hkv = k.shape[1]
    if k.shape != (S, Hkv, D) or v.shape != (S, Hkv, D) or plan.S != S:
        raise ValueError("attn_fwd: inconsistent shapes")
    qs, ks, vs = _shd(q, "q"), _shd(k, "k"), _shd(v, "v")
    lib = _lib.load()
    dev = q.device
    out = torch.empty((S, Hq, D), dtype=torch.bfloat16, device=dev)
    lse = torch.empty((Hq, S), dtype=torch.float32, device=dev)
    ws = _workspace(lib.artk_attn_fwd_workspace_bytes(S, Hkv, D), dev)
    scale = float(D) ** -0.5 if scale is None else float(scale)
    _lib.check(
        lib.artk_attn_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), plan.buf.data_ptr(), S, Hq, Hkv, D,
                          qs[0], qs[1], ks[0], ks[1], vs[0], vs[1], out.stride(0), out.stride(1), scale,
                          out.data_ptr(), lse.data_ptr(), ws.data_ptr(), ws.numel(), _stream(dev))
    )
    return out, lse


def attn_bwd(q, k, v, out, lse, d_out, plan: AttnPlan, scale: Optional[float] = None):
    """(dq, dk, dv) bf16, contiguous [S, H, D], for the upstream gradient d_out of attn_fwd's out."""
    import ctypes as C

    S, Hq, D = q.shape
    Hkv = k.shape[1]
    lib = _lib.load()
    dev = q.device
    dq = torch.empty((S, Hq, D), dtype=torch.bfloat16, device=dev)
    dk = torch.empty((S, Hkv, D), dtype=torch.bfloat16, device=dev)
    dv = torch.empty((S, Hkv, D), dtype=torch.bfloat16, device=dev)
    _need(lse, "lse", torch.float32, (Hq, S))
    strides = []
    for name, t in (("q", q), ("k", k), ("v", v), ("out", out), ("d_out", d_out), ("dq", dq), ("dk", dk),
                    ("dv", dv)):
        strides += list(_shd(t, name))
    arr = (C.c_int64 * 16)(*strides)
    ws = _workspace(lib.artk_attn_bwd_workspace_bytes(S, Hq, Hkv, D), dev)
    scale = float(D) ** -0.5 if scale is None else float(scale)
    _lib.check(
        lib.artk_attn_bwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr(),
                          d_out.data_ptr(), plan.buf.data_ptr(), S, Hq, Hkv, D, arr, scale, dq.data_ptr(),
                          dk.data_ptr(), dv.data_ptr(), ws.data_ptr(), ws.numel(), _stream(dev))
    )
    return dq, dk, dv


# -----------------------------------------------------------------------------
# NF4 base weights
# -----------------------------------------------------------------------------
def nf4_dequant(packed, absmax=None, absmax_q=None, code2=None, absmax2=None, offset: float = 0.0,
                blocksize: int = 64, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """bf16 [2 * packed.numel()] from NF4 codes (see artk_nf4_dequant)."""
    _need(packed, "packed", torch.uint8)
    n = packed.numel() * 2
    if absmax is not None:
        _need(absmax, "absmax", torch.float32, (n // blocksize,))
    else:
        _need(absmax_q, "absmax_q", torch.uint8, (n // blocksize,))
        _need(code2, "code2", torch.float32, (256,))
        _need(absmax2, "absmax2", torch.float32)
    if out is None:
        out = torch.empty(n, dtype=torch.bfloat16, device=packed.device)
    _lib.check(_lib.load().artk_nf4_dequant(packed.data_ptr(), _ptr(absmax), _ptr(absmax_q), _ptr(code2),
                                            _ptr(absmax2), offset, n, blocksize, out.data_ptr(),
                                            _stream(packed.device)))
    return out


def nf4_dequant_t(packed, rows: int, cols: int, absmax=None, absmax_q=None, code2=None, absmax2=None,
                  offset: float = 0.0, blocksize: int = 64) -> torch.Tensor:
    """bf16 [cols, rows]: the [rows, cols] weight behind the NF4 codes, written transposed."""
    _need(packed, "packed", torch.uint8, (rows * cols // 2,))
    out = torch.empty((cols, rows), dtype=torch.bfloat16, device=packed.device)
    _lib.check(_lib.load().artk_nf4_dequant_t(packed.data_ptr(), _ptr(absmax), _ptr(absmax_q), _ptr(code2),
                                              _ptr(absmax2), offset, rows, cols, blocksize, out.data_ptr(),
                                              _stream(packed.device)))
    return out


def _nf4_struct(w) -> "_lib.Nf4Struct":
    """artk_nf4_t for an art_amd.quant.NF4Weight (the tensors stay owned by `w`)."""
    n = w.shape[0] * w.shape[1]
    _need(w.packed, "packed", torch.uint8, (n // 2,))
    if w.absmax is not None:
        _need(w.absmax, "absmax", torch.float32, (n // w.blocksize,))
    else:
        _need(w.absmax_q, "absmax_q", torch.uint8, (n // w.blocksize,))
        _need(w.code2, "code2", torch.float32, (256,))
        _need(w.absmax2, "absmax2", torch.float32)
    return _lib.Nf4Struct(w.packed.data_ptr(), _ptr(w.absmax), _ptr(w.absmax_q), _ptr(w.code2), _ptr(w.absmax2),
                          float(w.offset), int(w.blocksize))


def _lora_proj_array(projs):
    """ctypes array of artk_lora_proj_t from dicts of tensors (missing keys: NULL)."""
    arr = (_lib.LoraProjStruct * len(projs))()
    for st, d in zip(arr, projs):
        for key in ("W", "W_t", "A", "B", "bias", "y", "g", "xa", "dA", "dB"):
            t = d.get(key)
            setattr(st, key, None if t is None else t.data_ptr())
        st.out, st.r = d["B"].shape
    return arr


def lora_linear_multi_fwd(x, Ws, As, Bs, scale: float, biases=None):
    """Projections of the same x in one call: for each i, (y_i bf16 [T,out_i], xa_i f32 [T,r_i]) with
    y_i = x W_i^T + bias_i + scale (x A_i^T) B_i^T.  Nothing is concatenated: every projection keeps
    its own weight, factors and output.  Returns (ys, xas)."""
    T, n_in = x.shape
    n = len(Ws)
    biases = biases if biases is not None else [None] * n
    _need(x, "x", torch.bfloat16)
    dev = x.device
    projs, ys, xas = [], [], []
    for W, A, B, bias in zip(Ws, As, Bs, biases):
        n_out, r = B.shape
        _need(W, "W", torch.bfloat16, (n_out, n_in))
        _need(A, "A", torch.bfloat16, (r, n_in))
        _need(B, "B", torch.bfloat16, (n_out, r))
        if bias is not None:
            _need(bias, "bias", torch.bfloat16, (n_out,))
        y = torch.empty((T, n_out), dtype=torch.bfloat16, device=dev)
        xa = torch.empty((T, r), dtype=torch.float32, device=dev)
        ys.append(y)
        xas.append(xa)
        projs.append({"W": W, "A": A, "B": B, "bias": bias, "y": y, "xa": xa})
    arr = _lora_proj_array(projs)
    lib = _lib.load()
    ws = _workspace(lib.artk_lora_linear_multi_fwd_workspace_bytes(T, n_in, arr, n), dev)
    _lib.check(lib.artk_lora_linear_multi_fwd(x.data_ptr(), arr, n, scale, T, n_in, ws.data_ptr(), ws.numel(),
                                              _stream(dev)))
    return ys, xas


def lora_linear_multi_bwd(gs, x, W_ts, As, Bs, xas, scale: float):
    """Backward of lora_linear_multi_fwd: (dx bf16 [T,in], [dA_i f32 [r_i,in]], [dB_i f32 [out_i,r_i]]) for
    the upstream gradients g_i bf16 [T,out_i]; dx is the sum over the projections."""
    T, n_in = x.shape
    n = len(gs)
    _need(x, "x", torch.bfloat16)
    dev = x.device
    projs, dAs, dBs = [], [], []
    for g, W_t, A, B, xa in zip(gs, W_ts, As, Bs, xas):
        n_out, r = B.shape
        _need(g, "g", torch.bfloat16, (T, n_out))
        _need(W_t, "W_t", torch.bfloat16, (n_in, n_out))
        _need(A, "A", torch.bfloat16, (r, n_in))
        _need(B, "B", torch.bfloat16, (n_out, r))
        _need(xa, "xa", torch.float32, (T, r))
        dA = torch.empty((r, n_in), dtype=torch.float32, device=dev)
        dB = torch.empty((n_out, r), dtype=torch.float32, device=dev)
        dAs.append(dA)
        dBs.append(dB)
        projs.append({"W_t": W_t, "A": A, "B": B, "g": g, "xa": xa, "dA": dA, "dB": dB})
    arr = _lora_proj_array(projs)
    lib = _lib.load()
    dx = torch.empty((T, n_in), dtype=torch.bfloat16, device=dev)
    ws = _workspace(lib.artk_lora_linear_multi_bwd_workspace_bytes(T, n_in, arr, n), dev)
    _lib.check(lib.artk_lora_linear_multi_bwd(x.data_ptr(), arr, n, scale, T, n_in, dx.data_ptr(), ws.data_ptr(),
                                              ws.numel(), _stream(dev)))
    return dx, dAs, dBs


def lora_linear_fwd_nf4(x, w_nf4, A, B, scale: float, bias: Optional[torch.Tensor] = None):
    """lora_linear_fwd with the frozen weight given as NF4 codes (art_amd.quant.NF4Weight); the
    bf16 weight lives in the call's workspace only."""
    import ctypes as C

    T, n_in = x.shape
    n_out, r = B.shape
    if tuple(w_nf4.shape) != (n_out, n_in):
        raise ValueError(f"NF4 weight has shape {tuple(w_nf4.shape)}, expected {(n_out, n_in)}")
    _need(x, "x", torch.bfloat16)
    _need(A, "A", torch.bfloat16, (r, n_in))
    _need(B, "B", torch.bfloat16, (n_out, r))
    if bias is not None:
        _need(bias, "bias", torch.bfloat16, (n_out,))
    lib = _lib.load()
    dev = x.device
    y = torch.empty((T, n_out), dtype=torch.bfloat16, device=dev)
    xa = torch.empty((T, r), dtype=torch.float32, device=dev)
    ws = _workspace(lib.artk_lora_linear_fwd_nf4_workspace_bytes(T, n_in, n_out, r), dev)
    st = _nf4_struct(w_nf4)
    _lib.check(lib.artk_lora_linear_fwd_nf4(x.data_ptr(), C.byref(st), A.data_ptr(), B.data_ptr(), _ptr(bias),
                                            scale, T, n_in, n_out, r, y.data_ptr(), xa.data_ptr(),
                                            ws.data_ptr(), ws.numel(), _stream(dev)))
    return y, xa


def lora_linear_bwd_nf4(g, x, w_nf4, A, B, xa, scale: float):
    """lora_linear_bwd with the frozen weight given as NF4 codes; no transposed copy is kept."""
    import ctypes as C

    T, n_in = x.shape
    n_out, r = B.shape
    _need(g, "g", torch.bfloat16, (T, n_out))
    _need(x, "x", torch.bfloat16)
    _need(A, "A", torch.bfloat16, (r, n_in))
    _need(B, "B", torch.bfloat16, (n_out, r))
    _need(xa, "xa", torch.float32, (T, r))
    lib = _lib.load()
    dev = x.device
    dx = torch.empty((T, n_in), dtype=torch.bfloat16, device=dev)
    dA = torch.empty((r, n_in), dtype=torch.float32, device=dev)
    dB = torch.empty((n_out, r), dtype=torch.float32, device=dev)
    ws = _workspace(lib.artk_lora_linear_bwd_nf4_workspace_bytes(T, n_in, n_out, r), dev)
    st = _nf4_struct(w_nf4)
    _lib.check(lib.artk_lora_linear_bwd_nf4(g.data_ptr(), x.data_ptr(), C.byref(st), A.data_ptr(), B.data_ptr(),
                                            xa.data_ptr(), scale, T, n_in, n_out, r, dx.data_ptr(),
                                            dA.data_ptr(), dB.data_ptr(), ws.data_ptr(), ws.numel(),
                                            _stream(dev)))
    return dx, dA, dB


# -----------------------------------------------------------------------------
# Optimizer
# -----------------------------------------------------------------------------
def sumsq(x: torch.Tensor) -> torch.Tensor:
    """f32 [1]: sum of squares of a flat f32 device tensor (fixed summation order)."""
    _need(x, "x", torch.float32)
    lib = _lib.load()
    out = torch.empty(1, dtype=torch.float32, device=x.device)
    ws = _workspace(lib.artk_sumsq_f32_workspace_bytes(), x.device)
    _lib.check(lib.artk_sumsq_f32(x.data_ptr(), x.numel(), out.data_ptr(), ws.data_ptr(), ws.numel(),
                                  _stream(x.device)))
    return out


def adamw_step(p, g, m, v, p_bf16, lr, beta1, beta2, eps, weight_decay, step, grad_sumsq=None,
               max_grad_norm=0.0) -> None:
    """In-place fused AdamW over flat f32 buffers (see artk_adamw_step)."""
    n = p.numel()
    for name, t in (("p", p), ("g", g), ("m", m), ("v", v)):
        _need(t, name, torch.float32)
        if t.numel() != n:
            raise ValueError(f"{name}: expected {n} elements")
    if p_bf16 is not None:
        _need(p_bf16, "p_bf16", torch.bfloat16)
    _lib.check(_lib.load().artk_adamw_step(p.data_ptr(), g.data_ptr(), m.data_ptr(), v.data_ptr(),
                                           _ptr(p_bf16), n, lr, beta1, beta2, eps, weight_decay, step,
                                           _ptr(grad_sumsq), max_grad_norm, _stream(p.device)))


def adamw8bit_step(p, g, state1, state2, absmax1, absmax2, qmap1, qmap2, p_bf16, lr, beta1, beta2, eps,
                   weight_decay, step, grad_sumsq=None, max_grad_norm=0.0) -> None:
    """In-place AdamW with 8-bit block-wise moments (see artk_adamw8bit_step)."""
    n = p.numel()
    nb = (n + 255) // 256
    _need(p, "p", torch.float32)
    _need(g, "g", torch.float32, (n,))
    _need(state1, "state1", torch.uint8, (n,))
    _need(state2, "state2", torch.uint8, (n,))
    _need(absmax1, "absmax1", torch.float32, (nb,))
    _need(absmax2, "absmax2", torch.float32, (nb,))
    _need(qmap1, "qmap1", torch.float32, (256,))
    _need(qmap2, "qmap2", torch.float32, (256,))
    if p_bf16 is not None:
        _need(p_bf16, "p_bf16", torch.bfloat16)
    _lib.check(_lib.load().artk_adamw8bit_step(
        p.data_ptr(), g.data_ptr(), state1.data_ptr(), state2.data_ptr(), absmax1.data_ptr(), absmax2.data_ptr(),
        qmap1.data_ptr(), qmap2.data_ptr(), _ptr(p_bf16), n, lr, beta1, beta2, eps, weight_decay, step,
        _ptr(grad_sumsq), max_grad_norm, _stream(p.device)))


# -----------------------------------------------------------------------------
# per-kernel timing
# -----------------------------------------------------------------------------
(PROF_LMHEAD_FWD, PROF_DHIDDEN_GEMM, PROF_TARGET_REF, PROF_LORA_GEMM, PROF_MOE_GEMM, PROF_ATTN_FWD,
 PROF_ATTN_BWD_KV, PROF_ATTN_BWD_Q) = range(8)


def profile_enable(on: bool) -> None:
    _lib.check(_lib.load().artk_profile_enable(int(on)))


def profile_collect(kind: int) -> Tuple[float, int]:
    """(summed milliseconds, launches) of one kernel kind; synchronise first."""
    import ctypes as C

    ms, n = C.c_double(0.0), C.c_int64(0)
    _lib.check(_lib.load().artk_profile_collect(kind, C.byref(ms), C.byref(n)))
    return ms.value, n.value


# -----------------------------------------------------------------------------
# ceilings of the part (measurement aids)
# -----------------------------------------------------------------------------
def mfma_loop(operands: torch.Tensor, iters: int, blocks: int, sink: Optional[torch.Tensor] = None,
              shape: str = "32x32x16") -> float:
    """Launches the MFMA-only loop (``shape``: "32x32x16", the main loop's instruction, or "16x16x32");
    returns the flop it executes (time it with events)."""
    _need(operands, "operands", torch.bfloat16)
    if shape not in ("32x32x16", "16x16x32"):
        raise ValueError("shape must be '32x32x16' or '16x16x32'")
    if sink is None:
        sink = torch.empty(blocks * 512, dtype=torch.float32, device=operands.device)
    _need(sink, "sink", torch.float32, (blocks * 512,))
    lib = _lib.load()
    fn = lib.artk_mfma_loop if shape == "32x32x16" else lib.artk_mfma_loop16
    _lib.check(fn(operands.data_ptr(), operands.numel(), int(iters), int(blocks), sink.data_ptr(),
                  _stream(operands.device)))
    return float(blocks) * 8 * iters * 32 * 32768.0


def stream_copy(src: torch.Tensor, dst: torch.Tensor) -> int:
    """dst = src with the library's plain copy kernel; returns the bytes copied."""
    if not (src.is_cuda and dst.is_cuda and src.is_contiguous() and dst.is_contiguous()):
        raise ValueError("src and dst must be contiguous GPU tensors")
    nbytes = src.numel() * src.element_size()
    if nbytes != dst.numel() * dst.element_size():
        raise ValueError("src and dst differ in size")
    _lib.check(_lib.load().artk_stream_copy(src.data_ptr(), dst.data_ptr(), nbytes, _stream(src.device)))
    return nbytes


def lds_probe(waves: int, kind: int, reads_per_dma: int, iters: int, blocks: int,
              device: torch.device) -> dict:
    """Runs the LDS bandwidth probe and synchronises.  ``kind``: 0 ds_read_b128 contiguous, 1 ds_read_b128
    in the GEMM's fragment pattern, 2 ds_read_b64_tr_b16.  Returns the read (and DMA-written) bytes per
    core clock and CU (median over the work-groups) and the core clock in GHz seen by the probe."""
    src = torch.zeros(65536, dtype=torch.uint8, device=device)
    cyc = torch.zeros(blocks, 2, dtype=torch.int64, device=device)
    _lib.check(_lib.load().artk_lds_probe(int(waves), int(kind), int(reads_per_dma), src.data_ptr(), int(iters),
                                          int(blocks), cyc.data_ptr(), _stream(device)))
    torch.cuda.synchronize(device)
    c = cyc.cpu()
    core = float(c[:, 0].median())
    ticks = float(c[:, 1].median())
    read_bytes = float(waves) * iters * 16 * (512 if kind == 2 else 1024)
    n_dma = 0 if reads_per_dma == 0 else len([j for j in range(16) if j % reads_per_dma == reads_per_dma - 1])
    write_bytes = float(waves) * iters * n_dma * 1024
    return {"read_B_per_clk": read_bytes / core, "dma_write_B_per_clk": write_bytes / core,
            "core_GHz": core / (ticks * 10.0) if ticks > 0 else None}


def gemm_loop_probe(p: torch.Tensor, q: torch.Tensor, loop: int = 0, ablate: int = 0, group: int = 8,
                    same_tile: bool = False, out: Optional[torch.Tensor] = None,
                    cycles: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out bf16 [N,M] = q [N,K] @ p [M,K]^T on a chosen main loop (0: 8-wave, every wave issues its own
    DMA; 5: 8-wave, the first wave of each SIMD issues the DMA of both; 1: 4-wave 32x32x16; 2: 4-wave
    16x16x32; 3: 8-wave 16x16x32; 4: 256 x 128 tiles with two work-groups per CU), tile-order group and
    ablation switches (see artk_gemm_loop_probe); the result is only meaningful with same_tile False and
    ablate == 0 (or loop 5, where ablate 1 is another correct variant)."""
    M, K = p.shape
    N = q.shape[0]
    _need(p, "p", torch.bfloat16)
    _need(q, "q", torch.bfloat16, (N, K))
    if out is None:
        out = torch.empty((N, M), dtype=torch.bfloat16, device=p.device)
    _need(out, "out", torch.bfloat16, (N, M))
    if cycles is not None:
        _need(cycles, "cycles", torch.int64)
        if cycles.numel() < 2 * torch.cuda.get_device_properties(p.device).multi_processor_count:
            raise ValueError("cycles needs two int64 per CU")
    _lib.check(_lib.load().artk_gemm_loop_probe(p.data_ptr(), q.data_ptr(), out.data_ptr(), M, N, K, int(loop),
                                                int(ablate), int(group), int(bool(same_tile)), _ptr(cycles),
                                                _stream(p.device)))
    return out
