/*
 * artk — C-ABI of the MI355X (gfx950) GRPO training hot path.
 *
 * Every entry point takes plain device pointers and sizes.  The caller owns all
 * memory (inputs, outputs and the workspace); the library holds no device
 * memory, launches on the stream it is given and never synchronises.
 *
 * Return value: 0 = ok, negative = argument error (ARTK_ERR_*), positive = the
 * hipError_t of a failed runtime call.  artk_last_error() returns a
 * thread-local message for the last non-zero return on the calling thread.
 *
 * Layouts: all matrices row-major and contiguous; bf16 = 16-bit brain float;
 * token ids int64; masks one byte per token (0 / 1); 16-byte aligned pointers.
 *
 * "shift": the reference scores position t against token t+1 by shifting every
 * per-token input one to the left with a pad value
 * (reference: src/art/local/train.py:284-285, used at :79 and :112-117).
 * With shift=1 the kernels read element t+1 of the un-shifted [B,S] input (pad
 * value at the last position of each row) instead of materialising shifted
 * copies; with shift=0 they read element t.
 */
#ifndef ARTK_H_
#define ARTK_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ARTK_OK 0
#define ARTK_ERR_INVALID_ARGUMENT (-1)
#define ARTK_ERR_WORKSPACE_TOO_SMALL (-2)
#define ARTK_ERR_UNSUPPORTED_SHAPE (-3)

typedef void* artk_stream_t; /* hipStream_t */

/* Library identification: ABI version (bumped on incompatible change). */
int32_t artk_abi_version(void);
const char* artk_last_error(void);

/* ------------------------------------------------------------------------- *
 * A2 — per-token logprob of the sampled token, forward only.
 * Replaces: src/art/local/train.py:245-281 (_calculate_logprobs: chunked
 *   matmul -> gather -> logsumexp -> subtract).  No [T,V] logits are written.
 *   hidden   bf16 [T,H]      (T = B*S positions)
 *   lm_head  bf16 [V,H]      (physical layout of the weight whose .t() the
 *                             reference passes, train.py:76-78)
 *   ids      int64 [T]       sampled token ids (see "shift"; pad id 0)
 *   logprob  f32 [T]  out    selected logit - logsumexp
 *   lse      f32 [T]  out    logsumexp (kept for the backward)
 * Requires H % 64 == 0, V % 8 == 0.  Ids outside [0,V) give NaN.
 * ------------------------------------------------------------------------- */
size_t artk_logprob_fwd_workspace_bytes(int64_t T, int64_t V, int64_t H);
int32_t artk_logprob_fwd(const void* hidden, const void* lm_head, const int64_t* ids, int32_t shift,
                         int64_t T, int64_t S, int64_t V, int64_t H, float* logprob, float* lse,
                         void* workspace, size_t workspace_bytes, artk_stream_t stream);

/* ------------------------------------------------------------------------- *
 * A7 (logprob part) — d_hidden[t,:] = g[t] * (W[y_t,:] - softmax(logits_t) W)
 * Replaces: autograd backward of train.py:265-272 w.r.t. hidden_states
 *   (lm_head is frozen: it is not a LoRA target, src/art/dev/model.py:54-62).
 *   lm_head_t  bf16 [H,V]   transposed copy of lm_head (artk_transpose_bf16)
 *   lse        f32 [T]      from artk_logprob_fwd
 *   grad_logprob f32 [T]    upstream gradient per position
 *   d_hidden   bf16 [T,H] out
 * Logits are recomputed per chunk of `chunk_tokens` positions into a bounded
 * bf16 scratch inside the workspace.  A row with a non-zero grad_logprob whose
 * target has probability below e^-80 gets a zero d_hidden row (see
 * artk_grpo_fused, which also counts such rows).  Requires H % 64 == 0, V % 64 == 0.
 * ------------------------------------------------------------------------- */
size_t artk_logprob_bwd_workspace_bytes(int64_t T, int64_t V, int64_t H, int64_t chunk_tokens);
int32_t artk_logprob_bwd(const void* hidden, const void* lm_head, const void* lm_head_t,
                         const int64_t* ids, int32_t shift, int64_t T, int64_t S, int64_t V,
                         int64_t H, const float* lse, const float* grad_logprob, void* d_hidden,
                         int64_t chunk_tokens, void* workspace, size_t workspace_bytes,
                         artk_stream_t stream);

/* ------------------------------------------------------------------------- *
 * A4 — GRPO clipped-surrogate loss on per-token logprobs, value + gradient.
 * Replaces: src/art/local/train.py:111-151 (shift, NaN-fill of old logprobs,
 *   ratio, clip, k3 KL, weight*mask, normalisation by mask.sum()+1e-6) and its
 *   autograd backward w.r.t. new_logprobs.
 *   new_logprob f32 [T]   (position frame, i.e. already "shifted")
 *   old_logprob f32 [T]   NaN = missing            (un-shifted if shift=1)
 *   advantages  f32 [T], weights f32 [T], mask u8 [T]   (same frame as old)
 *   ref_logprob f32 [T] or NULL (position frame; used when beta > 0)
 *   clip_lo / clip_hi     1-epsilon, 1+epsilon_high
 *   scalars f32 [4] out   {loss, mean_policy_loss, mean_kl, mask_count}
 *   coef    f32 [T] out   d loss / d new_logprob[t]   (may be NULL)
 * ------------------------------------------------------------------------- */
size_t artk_grpo_loss_workspace_bytes(int64_t T);
int32_t artk_grpo_loss(const float* new_logprob, const float* old_logprob, const float* advantages,
                       const uint8_t* mask, const float* weights, const float* ref_logprob,
                       int32_t shift, int64_t T, int64_t S, float clip_lo, float clip_hi, float beta,
                       float* scalars, float* coef, void* workspace, size_t workspace_bytes,
                       artk_stream_t stream);

/* ------------------------------------------------------------------------- *
 * artk_grpo_loss without a workspace argument and without any allocation.
 * No counterpart in the reference: it exists for callers that cannot allocate
 * (code under HIP graph capture, tight serving loops, harnesses that forbid the
 * allocator).  Same arguments, kernels and results as artk_grpo_loss; the
 * scratch (two f32 [T] arrays and a counter) lives in a device array inside the
 * library's code object (about 2 MiB per GPU the library runs on, held until
 * the process ends).  T above ARTK_GRPO_LOSS_STATIC_MAX_T is rejected with
 * ARTK_ERR_UNSUPPORTED_SHAPE.  The first call on a device looks up the array's
 * address (hipGetSymbolAddress) and should be made outside a capture.  All calls
 * on one GPU share the array: calls that overlap on one GPU (different streams
 * or threads) race; nothing in it has to start at zero (every element a call
 * reads is written by that call first).
 * ------------------------------------------------------------------------- */
#define ARTK_GRPO_LOSS_STATIC_MAX_T 262144
int32_t artk_grpo_loss_static(const float* new_logprob, const float* old_logprob, const float* advantages,
                              const uint8_t* mask, const float* weights, const float* ref_logprob,
                              int32_t shift, int64_t T, int64_t S, float clip_lo, float clip_hi,
                              float beta, float* scalars, float* coef, artk_stream_t stream);

/* ------------------------------------------------------------------------- *
 * A1+A2+A4+A7 fused — loss and d_hidden of one packed batch in one call.
 * Replaces: the body of compute_loss, src/art/local/train.py:76-151, plus the
 *   backward that HF Trainer.training_step triggers on its result.
 * Per chunk of `chunk_tokens` positions: lm_head GEMM with online log-sum-exp
 * and target gather (for the rows the backward will read, exp(logit - the
 * target's logit) goes to a bounded bf16 scratch), loss coefficients, d_hidden
 * GEMM of those exponentials against lm_head_t, softmax scaling and one-hot
 * term in its reduction.  A row whose target has probability below e^-80 under
 * the current policy (log-sum-exp more than 80 nats above the target's logit)
 * would overflow the scratch: its d_hidden row is written as zeros and it is
 * counted in scalars[4]; its logprob and its loss term are exact.  Every other
 * row's exponentials are finite by construction, so d_hidden is always finite.
 *   tokens int64 [T], old_logprob/advantages/weights f32 [T], mask u8 [T]:
 *     the un-shifted PackedTensors rows (src/art/local/pack.py:13-21);
 *     the shift of train.py:79,112-117 is applied by index arithmetic.
 *   ref_logprob f32 [T] or NULL   (position frame)
 *   scalars f32 [5] out: {loss, mean_policy_loss, mean_kl, mask_count, dropped_rows}
 *   logprob f32 [T] out, d_hidden bf16 [T,H] out
 *   flags: 0, or ARTK_FUSED_SKIP_INACTIVE: evaluate the lm_head projection only
 *     for positions that can contribute to the loss (shifted assistant mask set,
 *     weight != 0, and advantage != 0 or a KL term).  The reference computes
 *     logprobs for every position and multiplies the rest by a zero mask
 *     (train.py:111-151); loss, metrics and d_hidden are the same, but logprob
 *     of a skipped position is NaN.  Needs T*H*2 < 2^31.
 * Requires H % 64 == 0, V % 64 == 0.
 * ------------------------------------------------------------------------- */
#define ARTK_FUSED_SKIP_INACTIVE 1
size_t artk_grpo_fused_workspace_bytes(int64_t T, int64_t V, int64_t H, int64_t chunk_tokens);
int32_t artk_grpo_fused(const void* hidden, const void* lm_head, const void* lm_head_t,
                        const int64_t* tokens, const float* old_logprob, const float* advantages,
                        const uint8_t* mask, const float* weights, const float* ref_logprob,
                        int64_t T, int64_t S, int64_t V, int64_t H, float clip_lo, float clip_hi,
                        float beta, int64_t chunk_tokens, int32_t flags, float* scalars,
                        float* logprob, void* d_hidden, void* workspace, size_t workspace_bytes,
                        artk_stream_t stream);

/* out[c,r] = in[r,c] for a bf16 [R,C] matrix (R, C multiples of 8).  Used once
 * per frozen weight to build the K-contiguous operand of the backward GEMMs. */
int32_t artk_transpose_bf16(const void* in, void* out, int64_t R, int64_t C, artk_stream_t stream);

/* Plain NT GEMM out[n,m] (bf16 or f32) = sum_k Q[n,k] * P[m,k]; exposed for
 * tests and roofline measurement of the shared main loop.
 * K % 64 == 0, M % 4 == 0. out_f32: 0 -> bf16 output, 1 -> f32 output. */
int32_t artk_gemm_nt(const void* P, const void* Q, void* out, int64_t M, int64_t N, int64_t K,
                     int32_t out_f32, artk_stream_t stream);

/* ------------------------------------------------------------------------- *
 * A8 — LoRA linear:  y = x W^T + scale * (x A^T) B^T      (scale = alpha / r)
 * Replaces: the peft 0.15.2 lora.Linear forward that the reference installs on
 *   the seven projection modules (src/art/local/state.py:86-92,
 *   src/art/dev/model.py:52-67; arithmetic in the third-party package).
 *   x bf16 [T,in], W bf16 [out,in] (frozen), A bf16 [r,in], B bf16 [out,r]
 *   bias bf16 [out] or NULL: the frozen bias of the wrapped linear (Qwen2.5 has one on
 *        q/k/v; peft keeps the base layer's bias), added in the GEMM epilogue: y += bias
 *        (16-byte aligned like every other pointer: it is read with vector loads)
 *   y bf16 [T,out] out, xa f32 [T,r] out (x A^T, kept for the backward)
 * Requires in % 64 == 0, out % 64 == 0, r % 8 == 0, r <= 64.
 * ------------------------------------------------------------------------- */
size_t artk_lora_linear_fwd_workspace_bytes(int64_t T, int64_t in, int64_t out, int32_t r);
int32_t artk_lora_linear_fwd(const void* x, const void* W, const void* A, const void* B, const void* bias,
                             float scale, int64_t T, int64_t in, int64_t out, int32_t r, void* y, float* xa,
                             void* workspace, size_t workspace_bytes, artk_stream_t stream);

/* Backward of the above for upstream gradient g bf16 [T,out]:
 *   dx bf16 [T,in] = g W + scale (g B) A
 *   dA f32 [r,in]  = scale (g B)^T x        dB f32 [out,r] = scale g^T (x A^T)
 * Replaces: autograd of peft's lora.Linear (W frozen, so no dW).
 *   W_t bf16 [in,out]: transposed copy of W (artk_transpose_bf16); xa from the forward.
 * g is read from HBM once for g B and dB together (and once more by the dx GEMM), x once
 * for dA; the sums over column chunks / row slabs are taken in a fixed order.
 * xa, dA, dB 16-byte aligned. */
size_t artk_lora_linear_bwd_workspace_bytes(int64_t T, int64_t in, int64_t out, int32_t r);
int32_t artk_lora_linear_bwd(const void* g, const void* x, const void* W_t, const void* A,
                             const void* B, const float* xa, float scale, int64_t T, int64_t in,
                             int64_t out, int32_t r, void* dx, float* dA, float* dB, void* workspace,
                             size_t workspace_bytes, artk_stream_t stream);

/* ------------------------------------------------------------------------- *
 * A9 — MoE expert path (no counterpart in the reference at this commit; the
 * contract is the benchmark configuration: 128 experts, top-8, rank-8 LoRA per
 * expert, tokens permuted into expert-contiguous groups).
 *
 * artk_moe_route: top-k experts per token and the expert-contiguous permutation.
 *   router_logits f32 [T,E]
 *   topk_idx i32 [T,k]   experts by decreasing logit, ties to the lower index; a NaN
 *                        logit counts as -inf, so every index lies in [0,E) whatever the
 *                        row holds (ties among -inf also go to the lower index)
 *   topk_w   f32 [T,k]   softmax probabilities of the chosen experts, renormalised; an
 *                        expert at -inf gets 0, a row without any finite logit all 0
 *   perm     i32 [T*k]   perm[i] = flat (token*k + slot) index of sorted row i;
 *                        stable sort of the token-major list by expert id
 *   inv_perm i32 [T*k]   inverse of perm;  row_token i32 [T*k] = perm[i] / k
 *   expert_offsets i32 [E+1]  first sorted row of each expert
 *   tile_prefix, blk_prefix i32 [E+1]  work lists of the grouped kernels
 *     (prefix sums of ceil(rows_e/256) and ceil(rows_e/16))
 * ------------------------------------------------------------------------- */
size_t artk_moe_route_workspace_bytes(int64_t T, int32_t E, int32_t k);
int32_t artk_moe_route(const float* router_logits, int64_t T, int32_t E, int32_t k, int32_t* topk_idx,
                       float* topk_w, int32_t* perm, int32_t* inv_perm, int32_t* row_token,
                       int32_t* expert_offsets, int32_t* tile_prefix, int32_t* blk_prefix,
                       void* workspace, size_t workspace_bytes, artk_stream_t stream);

/* Per-expert LoRA linear over the sorted rows:
 *   y[i,:] = x[src(i),:] W_e^T + scale (x[src(i),:] A_e^T) B_e^T,  e = expert of row i
 *   src(i) = gather[i] when gather != NULL (rows of x picked by row_token), else i.
 *   W bf16 [E,out,in], A bf16 [E,r,in], B bf16 [E,out,r]
 *   y bf16 [n_rows,out] out, xa f32 [n_rows,r] out (kept for the backward)
 *   With a gather, n_rows * in * 2 bytes must stay below 2 GiB (31-bit offsets from x). */
size_t artk_moe_lora_grouped_fwd_workspace_bytes(int64_t n_rows, int64_t in, int64_t out, int32_t E,
                                                 int32_t r);
int32_t artk_moe_lora_grouped_fwd(const void* x, const int32_t* gather, const void* W, const void* A,
                                  const void* B, float scale, const int32_t* expert_offsets,
                                  const int32_t* tile_prefix, const int32_t* blk_prefix,
                                  int64_t n_rows, int64_t in, int64_t out, int32_t E, int32_t r,
                                  void* y, float* xa, void* workspace, size_t workspace_bytes,
                                  artk_stream_t stream);

/* Backward of the above for g bf16 [n_rows,out]:
 *   dx bf16 [n_rows,in] (per sorted row; the caller sums the k rows of a token)
 *   dA f32 [E,r,in], dB f32 [E,out,r];  W_t bf16 [E,in,out] (artk_transpose_bf16_batched) */
size_t artk_moe_lora_grouped_bwd_workspace_bytes(int64_t n_rows, int64_t in, int64_t out, int32_t E,
                                                 int32_t r);
int32_t artk_moe_lora_grouped_bwd(const void* g, const void* x, const int32_t* gather, const void* W_t,
                                  const void* A, const void* B, const float* xa, float scale,
                                  const int32_t* expert_offsets, const int32_t* tile_prefix,
                                  const int32_t* blk_prefix, int64_t n_rows, int64_t in, int64_t out,
                                  int32_t E, int32_t r, void* dx, float* dA, float* dB,
                                  void* workspace, size_t workspace_bytes, artk_stream_t stream);

/* out[b,c,r] = in[b,r,c] for n bf16 [R,C] matrices. */
int32_t artk_transpose_bf16_batched(const void* in, void* out, int64_t n, int64_t R, int64_t C,
                                    artk_stream_t stream);

/* ------------------------------------------------------------------------- *
 * Packed-row attention without the dense bias.
 * Replaces: calculate_attn_bias, src/art/local/train.py:177-215 (a dense
 *   [1,S,S] additive bias: 0 where  j <= i && (group[i] == group[j] ||
 *   parent[i] == group[j]),  -inf elsewhere) and the masked softmax attention
 *   of the model that consumes it as `causal_mask` (train.py:239-241; the
 *   attention itself is third-party model code).  group_ids / parent_ids are
 *   the PackedTensors rows of src/art/local/pack.py:13-21 (int64, pad -1).
 *
 * artk_attn_plan: once per packed row; the plan (device memory owned by the
 *   caller, artk_attn_plan_bytes(S) bytes) is shared by every layer and head.
 *   It holds int32 equality codes of the ids and, per block of queries, the
 *   list of key blocks with at least one visible pair.
 * artk_attn_fwd: out = softmax(scale * q k^T + bias) v, lse = log-sum-exp of
 *   the biased scores (natural log).  Element (s, h, d) of q is at
 *   q[s * q_stride_s + h * q_stride_h + d] (bf16; strides in elements,
 *   multiples of 8), likewise k, v ([S, Hkv, D]) and out; query head h reads
 *   key/value head h / (Hq / Hkv).  lse is f32 [Hq, S].
 * artk_attn_bwd: dq, dk, dv (bf16, same addressing as q, k, v) from d_out.
 * Requires S % 256 == 0, S <= 65536, D in {64, 128}, scale > 0 (forward).
 * ------------------------------------------------------------------------- */
size_t artk_attn_plan_bytes(int64_t S);
int32_t artk_attn_plan(const int64_t* group_ids, const int64_t* parent_ids, int64_t S, void* plan,
                       size_t plan_bytes, artk_stream_t stream);
size_t artk_attn_fwd_workspace_bytes(int64_t S, int32_t Hkv, int32_t D);
int32_t artk_attn_fwd(const void* q, const void* k, const void* v, const void* plan, int64_t S,
                      int32_t Hq, int32_t Hkv, int32_t D, int64_t q_stride_s, int64_t q_stride_h,
                      int64_t k_stride_s, int64_t k_stride_h, int64_t v_stride_s, int64_t v_stride_h,
                      int64_t o_stride_s, int64_t o_stride_h, float scale, void* out, float* lse,
                      void* workspace, size_t workspace_bytes, artk_stream_t stream);
/* strides: 16 element strides, (stride_s, stride_h) of q, k, v, out, d_out, dq, dk, dv in that order. */
size_t artk_attn_bwd_workspace_bytes(int64_t S, int32_t Hq, int32_t Hkv, int32_t D);
int32_t artk_attn_bwd(const void* q, const void* k, const void* v, const void* out, const float* lse,
                      const void* d_out, const void* plan, int64_t S, int32_t Hq, int32_t Hkv,
                      int32_t D, const int64_t* strides, float scale, void* dq, void* dk, void* dv,
                      void* workspace, size_t workspace_bytes, artk_stream_t stream);

/* Tuning aid of artk_attn_bwd (no counterpart in the reference).  With grouped-query heads a
 * key block seen by at most `light_max` (query tile, head) pairs is handled by one work-group
 * for all heads of its group; busier blocks get one work-group per head and a fixed-order
 * reduction.  The library picks the threshold by itself (64 for rows long enough to fill the
 * GPU that way, else 0); this call overrides it for later artk_attn_bwd calls made on the
 * calling thread, light_max < 0 restores the automatic choice.  Results agree to rounding. */
int32_t artk_attn_bwd_tuning(int32_t light_max);

/* ------------------------------------------------------------------------- *
 * Optimizer step over the adapter parameters kept in one flat fp32 buffer.
 * Replaces: the per-tensor AdamW step and gradient clipping that HF Trainer runs
 *   with the reference's settings, src/art/dev/model.py:69-85 (betas 0.9 / 0.99,
 *   weight_decay 0.1, max_grad_norm 0.1, constant lr; `paged_adamw_8bit` there:
 *   the moments are kept in fp32 here).
 * artk_sumsq_f32: out[0] = sum x[i]^2 (fixed summation order, double partials).
 * artk_adamw_step: g' = g * min(1, max_grad_norm / (sqrt(*grad_sumsq) + 1e-6))
 *   (no clipping when grad_sumsq is NULL); p *= 1 - lr * weight_decay;
 *   m = m + (g' - m)(1 - beta1); v = beta2 v + (1 - beta2) g'^2;
 *   p -= lr / (1 - beta1^step) * m / (sqrt(v) / sqrt(1 - beta2^step) + eps);
 *   params_bf16 (may be NULL) receives the rounded copy of p.  step counts from 1.
 * ------------------------------------------------------------------------- */
size_t artk_sumsq_f32_workspace_bytes(void);
int32_t artk_sumsq_f32(const float* x, int64_t n, float* out, void* workspace, size_t workspace_bytes,
                       artk_stream_t stream);
int32_t artk_adamw_step(float* params, const float* grads, float* exp_avg, float* exp_avg_sq,
                        void* params_bf16, int64_t n, float lr, float beta1, float beta2, float eps,
                        float weight_decay, int32_t step, const float* grad_sumsq, float max_grad_norm,
                        artk_stream_t stream);

/* The same step with the moments in the storage form of `paged_adamw_8bit`
 * (src/art/dev/model.py:75; the arithmetic is bitsandbytes' block-wise 8-bit optimizer, not in
 * the reference tree): one byte per element and moment, an index into a 256-entry ascending
 * code book (qmap1 for exp_avg, values in [-1,1]; qmap2 for exp_avg_sq, values in [0,1]),
 * times one f32 maximum per block of 256 elements (absmax1 / absmax2, f32 [ceil(n/256)],
 * zero before the first step).  Per block: dequantise, g' as above,
 *   m = beta1 m + (1 - beta1) g';  v = beta2 v + (1 - beta2) g'^2;
 *   p = (p - lr sqrt(1 - beta2^t) / (1 - beta1^t) * m / (sqrt(v) + sqrt(1 - beta2^t) eps)) (1 - lr weight_decay);
 * new block maxima of |m| and v, each moment stored as the nearest code of m / max (ties to
 * the lower code).  10 bytes of state and gradient traffic per parameter less than the f32 form. */
int32_t artk_adamw8bit_step(float* params, const float* grads, void* state1, void* state2, float* absmax1,
                            float* absmax2, const float* qmap1, const float* qmap2, void* params_bf16,
                            int64_t n, float lr, float beta1, float beta2, float eps, float weight_decay,
                            int32_t step, const float* grad_sumsq, float max_grad_norm,
                            artk_stream_t stream);

/* ------------------------------------------------------------------------- *
 * NF4 base weight -> bf16.
 * Replaces: the dequantisation that bitsandbytes performs in front of every
 *   frozen linear when the base model is loaded with `load_in_4bit=True`
 *   (src/art/dev/model.py:29); the result feeds artk_lora_linear_fwd/bwd.
 *   packed  u8 [n/2]   two codes per byte, first element in the high nibble
 *   absmax  f32 [n/blocksize], or NULL with the double-quantised form:
 *   absmax_q u8 [n/blocksize], code2 f32 [256], absmax2 f32 [ceil(n/blocksize/256)],
 *           offset:  absmax[b] = code2[absmax_q[b]] * absmax2[b / 256] + offset
 *   out_bf16 [n] = bf16(level[code] * absmax[block])
 * n must be a multiple of blocksize (a power of two >= 32; bitsandbytes uses 64).
 * ------------------------------------------------------------------------- */
int32_t artk_nf4_dequant(const void* packed, const float* absmax, const void* absmax_q,
                         const float* code2, const float* absmax2, float offset, int64_t n,
                         int32_t blocksize, void* out_bf16, artk_stream_t stream);
/* The same values written transposed: the codes are a [rows, cols] matrix (blocks run along a
 * row), out_bf16 is [cols, rows].  rows, cols multiples of 8. */
int32_t artk_nf4_dequant_t(const void* packed, const float* absmax, const void* absmax_q,
                           const float* code2, const float* absmax2, float offset, int64_t rows,
                           int64_t cols, int32_t blocksize, void* out_bf16, artk_stream_t stream);

/* ------------------------------------------------------------------------- *
 * LoRA linear whose frozen weight stays in its NF4 storage form.
 * Replaces: the 4-bit base linear + peft lora.Linear pair of a model loaded with
 *   `load_in_4bit=True` (src/art/dev/model.py:29): bitsandbytes dequantises the weight in
 *   front of every matmul and keeps no 16-bit copy.
 * Same arguments and results as artk_lora_linear_fwd / _bwd, bit for bit, for the bf16 values
 * that artk_nf4_dequant gives; the 16-bit weight exists only inside the call, in the
 * workspace (forward: [out,in]; backward: [in,out], dequantised transposed), so no bf16
 * copy and no transposed copy of W stay resident between calls.
 * ------------------------------------------------------------------------- */
typedef struct artk_nf4 {
  const void* packed;    /* u8 [out*in/2] */
  const float* absmax;   /* f32 [out*in/blocksize], or NULL with the double-quantised form: */
  const void* absmax_q;  /* u8 [out*in/blocksize] */
  const float* code2;    /* f32 [256] */
  const float* absmax2;  /* f32 [ceil(out*in/blocksize/256)] */
  float offset;
  int32_t blocksize;     /* power of two >= 32 that divides `in` */
} artk_nf4_t;
size_t artk_lora_linear_fwd_nf4_workspace_bytes(int64_t T, int64_t in, int64_t out, int32_t r);
int32_t artk_lora_linear_fwd_nf4(const void* x, const artk_nf4_t* W, const void* A, const void* B,
                                 const void* bias, float scale, int64_t T, int64_t in, int64_t out, int32_t r,
                                 void* y, float* xa, void* workspace, size_t workspace_bytes,
                                 artk_stream_t stream);
size_t artk_lora_linear_bwd_nf4_workspace_bytes(int64_t T, int64_t in, int64_t out, int32_t r);
int32_t artk_lora_linear_bwd_nf4(const void* g, const void* x, const artk_nf4_t* W, const void* A,
                                 const void* B, const float* xa, float scale, int64_t T, int64_t in,
                                 int64_t out, int32_t r, void* dx, float* dA, float* dB, void* workspace,
                                 size_t workspace_bytes, artk_stream_t stream);

/* ------------------------------------------------------------------------- *
 * A8, several projections of the same input in one call: q|k|v or gate|up of a
 * layer.  Replaces: the separate peft lora.Linear modules the reference installs
 *   on q_proj, k_proj, v_proj (and gate_proj, up_proj), which all read the same
 *   hidden states (target modules: src/art/dev/model.py:54-62, installed at
 *   src/art/local/state.py:86-92).  Each projection keeps its own weight, adapter,
 *   output and gradient arrays: nothing is concatenated, no block-diagonal B is built.
 * Forward: x A_i^T of all projections in one launch, then ONE persistent GEMM launch
 *   over the tiles of all projections (narrow k / v ride along with q instead of
 *   leaving most of the GPU idle).  Writes y_i and xa_i of every projection.
 * Backward: per projection one pass over g_i (g_i B_i and dB_i); ONE GEMM launch for
 *   dx = sum_i (g_i W_i + scale (g_i B_i) A_i), the projections being K segments of
 *   one accumulation, so dx is written once; ONE pass over x for all dA_i.
 *   Writes dx, dA_i, dB_i; the ranks may add up to 64 at most.
 * Fields a direction does not use may be NULL.  Same shape rules as the single
 * projection: in % 64 == 0, out_i % 64 == 0, r_i % 8 == 0; all pointers 16-byte aligned.
 * ------------------------------------------------------------------------- */
#define ARTK_LORA_MULTI_MAX 4
typedef struct artk_lora_proj {
  const void* W;    /* bf16 [out,in]  frozen weight                (forward)  */
  const void* W_t;  /* bf16 [in,out]  its transposed copy          (backward) */
  const void* A;    /* bf16 [r,in]                                 (both)     */
  const void* B;    /* bf16 [out,r]                                (both)     */
  const void* bias; /* bf16 [out] or NULL, frozen                  (forward)  */
  void* y;          /* bf16 [T,out]   out                          (forward)  */
  const void* g;    /* bf16 [T,out]   upstream gradient of y       (backward) */
  float* xa;        /* f32 [T,r]      x A^T: out of the forward, in of the backward */
  float* dA;        /* f32 [r,in]     out                          (backward) */
  float* dB;        /* f32 [out,r]    out                          (backward) */
  int64_t out;
  int32_t r;
} artk_lora_proj_t;
size_t artk_lora_linear_multi_fwd_workspace_bytes(int64_t T, int64_t in, const artk_lora_proj_t* proj,
                                                  int32_t n);
int32_t artk_lora_linear_multi_fwd(const void* x, const artk_lora_proj_t* proj, int32_t n, float scale,
                                   int64_t T, int64_t in, void* workspace, size_t workspace_bytes,
                                   artk_stream_t stream);
size_t artk_lora_linear_multi_bwd_workspace_bytes(int64_t T, int64_t in, const artk_lora_proj_t* proj,
                                                  int32_t n);
int32_t artk_lora_linear_multi_bwd(const void* x, const artk_lora_proj_t* proj, int32_t n, float scale,
                                   int64_t T, int64_t in, void* dx, void* workspace, size_t workspace_bytes,
                                   artk_stream_t stream);

/* ------------------------------------------------------------------------- *
 * Per-kernel timing (measurement aid; no counterpart in the reference).
 * artk_profile_enable(1) makes later calls bracket each dominant kernel with
 * HIP events on the launch stream; after the caller has synchronised,
 * artk_profile_collect(kind, ...) returns the summed duration and the launch
 * count of that kind; artk_profile_enable(0) frees the events and turns it off.
 * ------------------------------------------------------------------------- */
#define ARTK_PROF_LMHEAD_FWD 0
#define ARTK_PROF_DHIDDEN_GEMM 1
#define ARTK_PROF_TARGET_REF 2 /* the reference-logit pre-pass of a stashed chunk */
#define ARTK_PROF_LORA_GEMM 3
#define ARTK_PROF_MOE_GEMM 4
#define ARTK_PROF_ATTN_FWD 5
#define ARTK_PROF_ATTN_BWD_KV 6
#define ARTK_PROF_ATTN_BWD_Q 7
int32_t artk_profile_enable(int32_t on);
int32_t artk_profile_collect(int32_t kind, double* total_ms, int64_t* launches);

/* ------------------------------------------------------------------------- *
 * Ceilings of the part, measured rather than quoted (measurement aids; no
 * counterpart in the reference).
 * artk_mfma_loop: `blocks` work-groups of 8 waves; every wave keeps the register
 *   tile of the GEMM main loop (4 x 2 MFMA 32x32x16 bf16 tiles) and issues
 *   `iters` rounds of 32 MFMAs on fragments read once from `operands`
 *   (bf16 [n_operands], n_operands >= 4096, a multiple of 8); no LDS, no memory
 *   traffic inside the loop.  Work: blocks * 8 * iters * 32 * 32768 flop.
 *   sink f32 [blocks * 512] receives a checksum per lane.
 * artk_mfma_loop16: the same arguments and the same work per round as 64 MFMA
 *   16x16x32 instructions on 8 x 4 tiles of 16 x 16 per wave.
 * artk_stream_copy: dst[i] = src[i], 16 bytes per lane and step (bytes % 16 == 0).
 * artk_lds_probe: LDS bytes per clock of a CU.  `blocks` work-groups of `waves` (4 or 8)
 *   wavefronts; every wave issues `iters` rounds of 16 LDS reads whose results nothing
 *   consumes: kind 0 = ds_read_b128, 1 KiB contiguous per wave instruction; kind 1 =
 *   ds_read_b128 in the swizzled operand-fragment pattern of the GEMM main loop; kind 2 =
 *   ds_read_b64_tr_b16 (transposed read, 512 bytes per wave instruction).  reads_per_dma
 *   0: reads only; 2 or 3: one 1 KiB `buffer_load ... lds` write from `src` (64 KiB,
 *   16-byte aligned, stays in L2) into another part of LDS per that many reads, the mix
 *   of the 4-wave / 8-wave main loop.  cycles int64 [blocks][2] receives the core-clock
 *   cycles and the 100 MHz ticks each work-group spent in the loop (barrier to barrier); bytes read
 *   per work-group: waves * iters * 16 * (1024 | 512).
 * ------------------------------------------------------------------------- */
int32_t artk_mfma_loop(const void* operands, int64_t n_operands, int64_t iters, int32_t blocks,
                       float* sink, artk_stream_t stream);
int32_t artk_mfma_loop16(const void* operands, int64_t n_operands, int64_t iters, int32_t blocks,
                         float* sink, artk_stream_t stream);
int32_t artk_stream_copy(const void* src, void* dst, int64_t bytes, artk_stream_t stream);
/* artk_gemm_loop_probe: persistent plain NT GEMM out[n,m] = sum_k Q[n,k] P[m,k] (bf16 [N,M]; M, N
 *   multiples of 256, K of 64) on a choice of main loop and tile order, with switches that take
 *   parts of the loop away, to measure what each part costs under the part's power limit.
 *   loop 0: the library's 8-wave loop as the kernels with a gathered operand run it (every wave
 *   issues its own share of the L2 -> LDS DMA); 5: the same loop as the kernels with two plain
 *   operands run it (the first wave of each SIMD issues the DMA of both); 1: the 4-wave loop with
 *   pinned instruction order (all three MFMA 32x32x16); 2: a 4-wave loop on MFMA 16x16x32; 3: the
 *   8-wave shape on MFMA 16x16x32; 4: 256 x 128 tiles on 4 waves with a 3-stage ring of K = 32
 *   stages, two work-groups per CU (cycles then holds the first work-group of each pair).
 *   ablate (loops 2 and 3; results are then wrong; 6, and 3 with loop 3, are not built):
 *   bit 1 no fill of the LDS stages inside the loop, bit 2 no wait for the fill and no work-group
 *   barrier, bit 4 no LDS fragment reads.  With loop 5, ablate 1 instead selects the variant that
 *   requests the whole fill of a stage right after the barrier that frees its buffer (results
 *   correct).  group: row-operand tiles walked per column-operand tile
 *   by consecutive tile ids (the library uses 8, or 4 when the row operand streams from HBM).
 *   same_tile != 0: every work-group fetches the same 8 operand tiles whatever it computes, so every
 *   fetch hits in L2 (results wrong).  cycles int64 [work-groups][2] or NULL: core-clock cycles and
 *   100 MHz ticks each work-group ran (one work-group per CU). */
int32_t artk_gemm_loop_probe(const void* P, const void* Q, void* out, int64_t M, int64_t N, int64_t K,
                             int32_t loop, int32_t ablate, int32_t group, int32_t same_tile, int64_t* cycles,
                             artk_stream_t stream);
int32_t artk_lds_probe(int32_t waves, int32_t kind, int32_t reads_per_dma, const void* src, int64_t iters,
                       int32_t blocks, int64_t* cycles, artk_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* ARTK_H_ */
