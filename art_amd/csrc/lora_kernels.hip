// LoRA linear forward / backward for gfx950:
//   y  = x W^T + s (x A^T) B^T
//   dx = g W   + s (g B) A        dA = s (g B)^T x        dB = s g^T (x A^T)
// W [out,in] frozen bf16, A [r,in], B [out,r], s = alpha / r.
//
// The reference configures this layer (src/art/local/state.py:86-92,
// src/art/dev/model.py:52-67: r = 8, alpha = 16, seven target modules) and
// leaves the arithmetic to peft 0.15.2 / unsloth 2025.5.1; the formulas above
// are those packages' documented LoRA linear.
//
// The dense products run on the shared 256x256 MFMA main loop.  The rank-r
// products ride along as extra K = 16 MFMA steps whose operands (the padded
// low-rank factors) are read straight from global memory, so y and dx are each
// one GEMM launch.  The skinny products (x A^T, g B: reductions along a row;
// dA, dB: reductions along the token axis) are bandwidth-bound helpers.
#include "common.hpp"
#include "gemm_nt.hpp"
#include "lora_common.hpp"

namespace artk {

// ----------------------------------------------------------------------------
// out[n, m] = sum_k Q[n,k] P[m,k] + sum_e Qe[n,e] Pe[m,e]     (bf16 out)
// ----------------------------------------------------------------------------
struct LoraGemmParams {
  const void* P;    // [M,K] row operand (weight)
  const void* Q;    // [N,K] column operand (activations)
  const uint16_t* Pe;  // [M,RP] low-rank factor of the row operand, or nullptr
  const uint16_t* Qe;  // [N,RP] low-rank factor of the column operand (scale folded in)
  uint16_t* out;    // [N,M]
  int64_t M, N, K;
  int RP, MT, NT;
};

__global__ __launch_bounds__(NTHREADS) void lora_gemm_kernel(LoraGemmParams p) {
  __shared__ __attribute__((aligned(1024))) char smem[GEMM_LDS_BYTES];
  const int id = xcd_remap(blockIdx.x, gridDim.x);
  int mt, nt;
  tile_coords(id, p.MT, p.NT, mt, nt);
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int half = lane >> 5;

  TileAcc acc;
  acc.zero();
  gemm_tile_nt(acc, smem, p.P, p.K, (int64_t)mt * TILE, p.M, p.Q, p.K, (int64_t)nt * TILE, p.N, 0,
               (int)p.K);

  if (p.Pe != nullptr) {
    // Rank-r part: operand fragments in MFMA layout come straight from global
    // memory (16 bytes per lane: row = lane % 32, 8 consecutive e per half-wave).
    int64_t prow[4], qrow[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      int64_t r = (int64_t)mt * TILE + wm * 128 + i * 32 + (lane & 31);
      prow[i] = r < p.M ? r : p.M - 1;
      int64_t c = (int64_t)nt * TILE + wn * 128 + i * 32 + (lane & 31);
      qrow[i] = c < p.N ? c : p.N - 1;
    }
    for (int e0 = 0; e0 < p.RP; e0 += 16) {
      Frags f;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        f.p[i] = *(const bf16x8*)(p.Pe + prow[i] * p.RP + e0 + half * 8);
        f.q[i] = *(const bf16x8*)(p.Qe + qrow[i] * p.RP + e0 + half * 8);
      }
      mma_frags(acc, f);
    }
  }

#pragma unroll
  for (int ni = 0; ni < 4; ++ni) {
    const int64_t col = (int64_t)nt * TILE + acc_col(wn, ni, lane);
    if (col >= p.N) continue;
#pragma unroll
    for (int mi = 0; mi < 4; ++mi)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int64_t m = (int64_t)mt * TILE + wm * 128 + mi * 32 + q * 8 + half * 4;
        if (m >= p.M) continue;
        bf16x4 o;
#pragma unroll
        for (int e = 0; e < 4; ++e) o[e] = (__bf16)acc.c[mi][ni][q * 4 + e];
        *(bf16x4*)(p.out + col * p.M + m) = o;
      }
  }
}

// ----------------------------------------------------------------------------
// Row products: out[t, j] = sum_k X[t,k] Mt[j,k] for the 16 rows j0..j0+15 of
// Mt (zero-padded factor, [RP,K]).  MFMA 16x16x32; a block owns 16 rows of X
// and its 4 waves split K.  Writes f32 [T,R] (unscaled) and bf16 [T,RP] (scaled).
// ----------------------------------------------------------------------------
__global__ __launch_bounds__(256) void rowdot16_kernel(const uint16_t* __restrict__ X,
                                                       const uint16_t* __restrict__ Mt, int64_t T,
                                                       int64_t K, int R, int RP, float scale,
                                                       float* __restrict__ out_f32,
                                                       uint16_t* __restrict__ out_bf16) {
  __shared__ floatx4 red[3][64];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int64_t t0 = (int64_t)blockIdx.x * 16;
  const int j0 = blockIdx.y * 16;
  int64_t trow = t0 + (lane & 15);
  if (trow >= T) trow = T - 1;
  const uint16_t* xp = X + trow * K + (lane >> 4) * 8;
  const uint16_t* mp = Mt + (int64_t)(j0 + (lane & 15)) * K + (lane >> 4) * 8;
  floatx4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
  for (int64_t k = (int64_t)wave * 32; k < K; k += 128) {
    bf16x8 a = *(const bf16x8*)(xp + k);
    bf16x8 b = *(const bf16x8*)(mp + k);
    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc, 0, 0, 0);
  }
  if (wave > 0) red[wave - 1][lane] = acc;
  __syncthreads();
  if (wave == 0) {
    acc += red[0][lane];
    acc += red[1][lane];
    acc += red[2][lane];
    // lane holds column j = lane % 16 of rows (lane / 16) * 4 + e
    const int j = j0 + (lane & 15);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int64_t t = t0 + (lane >> 4) * 4 + e;
      if (t < T) {
        if (j < R) out_f32[t * R + j] = acc[e];
        out_bf16[t * RP + j] = f32_to_bf16(acc[e] * scale);
      }
    }
  }
}

// ----------------------------------------------------------------------------
// Column products over a slab of rows:
//   partial[slab][c][r] = sum_{t in slab} X[t,c] Y[t,r]     r in [r0, r0+8)
// X [T,C] bf16, Y [T,R] f32.  A thread owns 4 columns; Y rows are staged in LDS
// and read as broadcasts.
// ----------------------------------------------------------------------------
constexpr int COLDOT_ROWS = 128;

__global__ __launch_bounds__(256) void coldot8_kernel(const uint16_t* __restrict__ X,
                                                      const float* __restrict__ Y, int64_t T,
                                                      int64_t C, int R, float* __restrict__ partial) {
  __shared__ float ys[COLDOT_ROWS][8];
  const int64_t c = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
  const int slab = blockIdx.y;
  const int r0 = blockIdx.z * 8;
  const int64_t t0 = (int64_t)slab * COLDOT_ROWS;
  const int nrows = (int)((T - t0) < COLDOT_ROWS ? (T - t0) : COLDOT_ROWS);
  for (int i = threadIdx.x; i < COLDOT_ROWS * 8; i += 256) {
    int rr = i >> 3, e = i & 7;
    ys[rr][e] = rr < nrows ? Y[(t0 + rr) * R + r0 + e] : 0.f;
  }
  __syncthreads();
  if (c >= C) return;
  float acc[4][8];
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[j][e] = 0.f;
  const uint16_t* xp = X + t0 * C + c;
#pragma unroll 4
  for (int rr = 0; rr < nrows; ++rr) {
    const uint2 raw = *(const uint2*)(xp + (int64_t)rr * C);
    const float x0 = __uint_as_float(raw.x << 16), x1 = __uint_as_float(raw.x & 0xffff0000u);
    const float x2 = __uint_as_float(raw.y << 16), x3 = __uint_as_float(raw.y & 0xffff0000u);
    const floatx4 ya = *(const floatx4*)&ys[rr][0];
    const floatx4 yb = *(const floatx4*)&ys[rr][4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      acc[0][e] += x0 * ya[e];
      acc[1][e] += x1 * ya[e];
      acc[2][e] += x2 * ya[e];
      acc[3][e] += x3 * ya[e];
      acc[0][4 + e] += x0 * yb[e];
      acc[1][4 + e] += x1 * yb[e];
      acc[2][4 + e] += x2 * yb[e];
      acc[3][4 + e] += x3 * yb[e];
    }
  }
  float* pp = partial + ((int64_t)slab * C + c) * R + r0;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    *(floatx4*)(pp + (int64_t)j * R) = floatx4{acc[j][0], acc[j][1], acc[j][2], acc[j][3]};
    *(floatx4*)(pp + (int64_t)j * R + 4) = floatx4{acc[j][4], acc[j][5], acc[j][6], acc[j][7]};
  }
}

// out = scale * sum over slabs; out is [C,R], or [R,C] when transpose_out.
__global__ __launch_bounds__(256) void coldot_reduce_kernel(const float* __restrict__ partial,
                                                            int nslab, int64_t C, int R, float scale,
                                                            int transpose_out,
                                                            float* __restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= C * R) return;
  float s = 0.f;
  for (int k = 0; k < nslab; ++k) s += partial[(int64_t)k * C * R + i];
  s *= scale;
  if (transpose_out) {
    const int64_t c = i / R;
    const int r = (int)(i - c * R);
    out[(int64_t)r * C + c] = s;
  } else {
    out[i] = s;
  }
}

static int32_t check_lora(int64_t T, int64_t in, int64_t out, int r) {
  ARTK_CHECK_ARG(T > 0 && in > 0 && out > 0 && r > 0, "T, in, out, r must be positive");
  if (in % BK != 0 || out % BK != 0) {
    set_error("in (%lld) and out (%lld) must be multiples of %d", (long long)in, (long long)out, BK);
    return ARTK_ERR_UNSUPPORTED_SHAPE;
  }
  if (r % 8 != 0 || r > 64) {
    set_error("LoRA rank %d must be a multiple of 8 and at most 64", r);
    return ARTK_ERR_UNSUPPORTED_SHAPE;
  }
  return ARTK_OK;
}

static int32_t launch_lora_gemm(const void* P, const void* Q, const uint16_t* Pe, const uint16_t* Qe,
                                void* out, int64_t M, int64_t N, int64_t K, int RP, hipStream_t st) {
  LoraGemmParams p;
  p.P = P;
  p.Q = Q;
  p.Pe = Pe;
  p.Qe = Qe;
  p.out = (uint16_t*)out;
  p.M = M;
  p.N = N;
  p.K = K;
  p.RP = RP;
  p.MT = (int)((M + TILE - 1) / TILE);
  p.NT = (int)((N + TILE - 1) / TILE);
  prof_begin(PROF_LORA_GEMM, st);
  lora_gemm_kernel<<<(unsigned)(p.MT * p.NT), NTHREADS, 0, st>>>(p);
  prof_end(PROF_LORA_GEMM, st);
  ARTK_CHECK_LAUNCH();
  return ARTK_OK;
}

// out_f32 [T,R] = X Mt^T (unscaled), out_bf16 [T,RP] = scale * that, zero padded.
static int32_t launch_rowdot(const void* X, const uint16_t* Mt_pad, int64_t T, int64_t K, int R,
                             int RP, float scale, float* out_f32, uint16_t* out_bf16,
                             hipStream_t st) {
  dim3 grid((unsigned)((T + 15) / 16), (unsigned)(RP / 16));
  rowdot16_kernel<<<grid, 256, 0, st>>>((const uint16_t*)X, Mt_pad, T, K, R, RP, scale, out_f32,
                                        out_bf16);
  ARTK_CHECK_LAUNCH();
  return ARTK_OK;
}

static int coldot_slabs(int64_t T) { return (int)((T + COLDOT_ROWS - 1) / COLDOT_ROWS); }

// out = scale * X^T Y  ([C,R], or [R,C] when transpose_out); X [T,C] bf16, Y [T,R] f32.
static int32_t launch_coldot(const void* X, const float* Y, int64_t T, int64_t C, int R, float scale,
                             int transpose_out, float* partial, float* out, hipStream_t st) {
  const int nslab = coldot_slabs(T);
  dim3 grid((unsigned)((C / 4 + 255) / 256), (unsigned)nslab, (unsigned)(R / 8));
  coldot8_kernel<<<grid, 256, 0, st>>>((const uint16_t*)X, Y, T, C, R, partial);
  ARTK_CHECK_LAUNCH();
  const int64_t n = C * R;
  coldot_reduce_kernel<<<(unsigned)((n + 255) / 256), 256, 0, st>>>(partial, nslab, C, R, scale,
                                                                    transpose_out, out);
  ARTK_CHECK_LAUNCH();
  return ARTK_OK;
}

}  // namespace artk

using namespace artk;

extern "C" {

size_t artk_lora_linear_fwd_workspace_bytes(int64_t T, int64_t in, int64_t out, int32_t r) {
  const int RP = round16(r);
  Workspace ws(nullptr, 0);
  ws.take<uint16_t>((size_t)RP * in);   // A padded [RP,in]
  ws.take<uint16_t>((size_t)out * RP);  // B padded [out,RP]
  ws.take<uint16_t>((size_t)T * RP);    // s * x A^T, bf16 [T,RP]
  return ws.used + 256;
}

int32_t artk_lora_linear_fwd(const void* x, const void* W, const void* A, const void* B, float scale,
                             int64_t T, int64_t in, int64_t out, int32_t r, void* y, float* xa,
                             void* workspace, size_t workspace_bytes, artk_stream_t stream) {
  int32_t rc = check_lora(T, in, out, r);
  if (rc) return rc;
  ARTK_CHECK_ARG(x && W && A && B && y && xa, "null pointer argument");
  ARTK_CHECK_ARG(aligned16(x) && aligned16(W) && aligned16(y), "pointers must be 16-byte aligned");
  const int RP = round16(r);
  Workspace ws(workspace, workspace_bytes);
  uint16_t* A16 = ws.take<uint16_t>((size_t)RP * in);
  uint16_t* B16 = ws.take<uint16_t>((size_t)out * RP);
  uint16_t* xa16 = ws.take<uint16_t>((size_t)T * RP);
  if (!ws.ok()) {
    set_error("workspace too small: need %zu bytes, got %zu", ws.used, workspace_bytes);
    return ARTK_ERR_WORKSPACE_TOO_SMALL;
  }
  hipStream_t st = (hipStream_t)stream;
  if ((rc = launch_pad(A, 1, r, in, 0, A16, RP, in, st))) return rc;
  if ((rc = launch_pad(B, 1, out, r, 0, B16, out, RP, st))) return rc;
  if ((rc = launch_rowdot(x, A16, T, in, r, RP, scale, xa, xa16, st))) return rc;
  return launch_lora_gemm(W, x, B16, xa16, y, out, T, in, RP, st);
}

size_t artk_lora_linear_bwd_workspace_bytes(int64_t T, int64_t in, int64_t out, int32_t r) {
  const int RP = round16(r);
  Workspace ws(nullptr, 0);
  ws.take<uint16_t>((size_t)RP * out);  // B^T padded [RP,out]
  ws.take<uint16_t>((size_t)in * RP);   // A^T padded [in,RP]
  ws.take<float>((size_t)T * r);        // g B, f32 [T,r]
  ws.take<uint16_t>((size_t)T * RP);    // s * g B, bf16 [T,RP]
  const int64_t widest = in > out ? in : out;
  ws.take<float>((size_t)coldot_slabs(T) * widest * r);
  return ws.used + 256;
}

int32_t artk_lora_linear_bwd(const void* g, const void* x, const void* W_t, const void* A,
                             const void* B, const float* xa, float scale, int64_t T, int64_t in,
                             int64_t out, int32_t r, void* dx, float* dA, float* dB, void* workspace,
                             size_t workspace_bytes, artk_stream_t stream) {
  int32_t rc = check_lora(T, in, out, r);
  if (rc) return rc;
  ARTK_CHECK_ARG(g && x && W_t && A && B && xa && dx && dA && dB, "null pointer argument");
  ARTK_CHECK_ARG(aligned16(g) && aligned16(x) && aligned16(W_t) && aligned16(dx),
                 "pointers must be 16-byte aligned");
  const int RP = round16(r);
  Workspace ws(workspace, workspace_bytes);
  uint16_t* Bt16 = ws.take<uint16_t>((size_t)RP * out);
  uint16_t* At16 = ws.take<uint16_t>((size_t)in * RP);
  float* gb = ws.take<float>((size_t)T * r);
  uint16_t* gb16 = ws.take<uint16_t>((size_t)T * RP);
  const int64_t widest = in > out ? in : out;
  float* partial = ws.take<float>((size_t)coldot_slabs(T) * widest * r);
  if (!ws.ok()) {
    set_error("workspace too small: need %zu bytes, got %zu", ws.used, workspace_bytes);
    return ARTK_ERR_WORKSPACE_TOO_SMALL;
  }
  hipStream_t st = (hipStream_t)stream;
  if ((rc = launch_pad(B, 1, out, r, 1, Bt16, RP, out, st))) return rc;
  if ((rc = launch_pad(A, 1, r, in, 1, At16, in, RP, st))) return rc;
  // g B  -> gb (f32) and s * gb (bf16, padded)
  if ((rc = launch_rowdot(g, Bt16, T, out, r, RP, scale, gb, gb16, st))) return rc;
  // dx = g W + (s g B) A
  if ((rc = launch_lora_gemm(W_t, g, At16, gb16, dx, in, T, out, RP, st))) return rc;
  // dA [r,in] = s (g B)^T x ;  dB [out,r] = s g^T (x A^T)
  if ((rc = launch_coldot(x, gb, T, in, r, scale, 1, partial, dA, st))) return rc;
  return launch_coldot(g, xa, T, out, r, scale, 0, partial, dB, st);
}

}  // extern "C"
