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
// products ride along as extra K = 16 MFMA steps whose operands (the low-rank
// factors) are read straight from global memory, so y and dx are each one GEMM
// launch.  The skinny products are bandwidth-bound: x A^T in the forward is a row
// product (rowdot16_kernel); in the backward g B and dB come from one pass over g
// and dA from one pass over x (lora_stats_kernel, skinny_stats.hpp).
#include "common.hpp"
#include "gemm_nt.hpp"
#include "lora_common.hpp"
#include "skinny_stats.hpp"

namespace artk {

constexpr int LORA_NI = 2;  // 8 waves, 2 per SIMD (see gemm_nt.hpp)

// ----------------------------------------------------------------------------
// out[n, m] = sum_k Q[n,k] P[m,k] + sum_e Qe[n,e] Pe[m,e]     (bf16 out)
// ----------------------------------------------------------------------------
struct LoraGemmParams {
  const void* P;       // [M,K] row operand (weight)
  const void* Q;       // [N,K] column operand (activations)
  const uint16_t* Pe;  // [M,r] low-rank factor of the row operand, or nullptr
  const uint16_t* Qe;  // [N,RP] low-rank factor of the column operand (scale folded in, zero padded)
  const uint16_t* bias;  // [M] added to every output row, or nullptr
  uint16_t* out;       // [N,M]
  int64_t M, N, K;
  int r, RP, MT, NT;
};

// Rank-r steps and bf16 store of one finished tile.
__device__ __forceinline__ void lora_gemm_epilogue(TileAcc<LORA_NI>& acc, const LoraGemmParams& p, int mt,
                                                   int nt) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int wm = wave_m<LORA_NI>(wave), wn = wave_n<LORA_NI>(wave);
  const int half = lane >> 5;
  if (p.Pe != nullptr) {
    int64_t prow[4], qrow[LORA_NI];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      int64_t r = (int64_t)mt * TILE + wm * 128 + i * 32 + (lane & 31);
      prow[i] = r < p.M ? r : p.M - 1;
    }
#pragma unroll
    for (int i = 0; i < LORA_NI; ++i) {
      int64_t c = (int64_t)nt * TILE + acc_col<LORA_NI>(wn, i, lane);
      qrow[i] = c < p.N ? c : p.N - 1;
    }
    lowrank_steps(acc, p.Pe, p.r, p.r, prow, p.Qe, p.RP, p.RP, qrow, p.RP);
  }
  if (p.bias != nullptr) {
    // element j of tile mi is output feature m0 + (j / 4) 8 + 4 half + j % 4
#pragma unroll
    for (int mi = 0; mi < 4; ++mi) {
      const int64_t m0 = (int64_t)mt * TILE + wm * 128 + mi * 32;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        int64_t mq = m0 + q * 8 + half * 4;
        mq = mq + 4 <= p.M ? mq : 0;  // rows past the end are never stored
        const bf16x4 bv = *(const bf16x4*)(p.bias + mq);
#pragma unroll
        for (int ni = 0; ni < LORA_NI; ++ni)
#pragma unroll
          for (int e = 0; e < 4; ++e) acc.c[mi][ni][q * 4 + e] += (float)bv[e];
      }
    }
  }

#pragma unroll
  for (int ni = 0; ni < LORA_NI; ++ni) {
    // lanes l and l + 32 share the column, so they take these branches together
    // (store_block_bf16 exchanges data between them)
    const int64_t col = (int64_t)nt * TILE + acc_col<LORA_NI>(wn, ni, lane);
    const bool col_ok = col < p.N;
#pragma unroll
    for (int mi = 0; mi < 4; ++mi) {
      const int64_t m0 = (int64_t)mt * TILE + wm * 128 + mi * 32;
      if (m0 >= p.M) continue;  // wave-uniform
      if (m0 + 32 <= p.M) {
        if (col_ok) store_block_bf16(p.out + col * p.M + m0, acc.c[mi][ni], half);
      } else {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int64_t m = m0 + q * 8 + half * 4;
          if (m >= p.M || !col_ok) continue;
          bf16x4 o;
#pragma unroll
          for (int e = 0; e < 4; ++e) o[e] = (__bf16)acc.c[mi][ni][q * 4 + e];
          *(bf16x4*)(p.out + col * p.M + m) = o;
        }
      }
    }
  }
}

// Persistent work-groups: tiles t, t + grid, ...; the first DMA stage of the next
// tile is started before the rank-r steps and the store of the current one.
__global__ __launch_bounds__(nthreads<LORA_NI>()) void lora_gemm_kernel(LoraGemmParams p) {
  __shared__ __attribute__((aligned(1024))) char smem[GEMM_LDS_BYTES];
  const int n_tiles = p.MT * p.NT;
  int t = blockIdx.x;
  int mt, nt;
  tile_coords(xcd_remap(t, n_tiles), p.MT, p.NT, mt, nt);
  {
    TileLoaders<LORA_NI> first;
    first.init(p.P, p.K, (int64_t)mt * TILE, p.M, p.Q, p.K, (int64_t)nt * TILE, p.N, 0, (int)p.K);
    first.issue_first(smem);
  }
  for (;;) {
    const int t2 = t + gridDim.x;
    const bool more = t2 < n_tiles;
    int mt2 = 0, nt2 = 0;
    if (more) tile_coords(xcd_remap(t2, n_tiles), p.MT, p.NT, mt2, nt2);
    TileAcc<LORA_NI> acc;
    acc.zero();
    {
      TileLoaders<LORA_NI> cur;  // its first stage is already on the way
      cur.init(p.P, p.K, (int64_t)mt * TILE, p.M, p.Q, p.K, (int64_t)nt * TILE, p.N, 0, (int)p.K);
      gemm_tile_run(acc, smem, cur);
    }
    if (more) {
      TileLoaders<LORA_NI> nxt;
      nxt.init(p.P, p.K, (int64_t)mt2 * TILE, p.M, p.Q, p.K, (int64_t)nt2 * TILE, p.N, 0, (int)p.K);
      nxt.issue_first(smem);
    }
    lora_gemm_epilogue(acc, p, mt, nt);
    if (!more) break;
    t = t2;
    mt = mt2;
    nt = nt2;
  }
}

// ----------------------------------------------------------------------------
// Row products: out[t, j] = sum_k X[t,k] Mt[j,k], Mt [R,K].  A block owns 16 rows
// of X and 16 rows j0..j0+15 of Mt (rows >= R read as zero); its 4 waves split K.
// Writes f32 [T,R] (unscaled) and bf16 [T,RP] (scaled, zero padded to RP).
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
  const int jm = j0 + (lane & 15);
  const uint16_t* xp = X + trow * K + (lane >> 4) * 8;
  const uint16_t* mp = Mt + (int64_t)(jm < R ? jm : 0) * K + (lane >> 4) * 8;
  floatx4 acc = rowdot_accumulate(xp, mp, jm < R, K, wave);
  acc = rowdot_block_sum(acc, red);
  if (wave == 0) {
    // lane holds column j = lane % 16 of rows (lane / 16) * 4 + e
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int64_t t = t0 + (lane >> 4) * 4 + e;
      if (t < T) {
        if (jm < R) out_f32[t * R + jm] = acc[e];
        out_bf16[t * RP + jm] = f32_to_bf16(acc[e] * scale);
      }
    }
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
                                const uint16_t* bias, void* out, int64_t M, int64_t N, int64_t K, int r,
                                int RP, hipStream_t st) {
  LoraGemmParams p;
  p.P = P;
  p.Q = Q;
  p.Pe = Pe;
  p.Qe = Qe;
  p.bias = bias;
  p.out = (uint16_t*)out;
  p.M = M;
  p.N = N;
  p.K = K;
  p.r = r;
  p.RP = RP;
  p.MT = (int)((M + TILE - 1) / TILE);
  p.NT = (int)((N + TILE - 1) / TILE);
  prof_begin(PROF_LORA_GEMM, st);
  {
    int cus = 0, dev = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
      cus = 256;
    const int n_tiles = p.MT * p.NT;
    lora_gemm_kernel<<<(unsigned)(n_tiles < cus ? n_tiles : cus), nthreads<LORA_NI>(), 0, st>>>(p);
  }
  prof_end(PROF_LORA_GEMM, st);
  ARTK_CHECK_LAUNCH();
  return ARTK_OK;
}

// out_f32 [T,R] = X Mt^T (unscaled), out_bf16 [T,RP] = scale * that, zero padded.
static int32_t launch_rowdot(const void* X, const void* Mt, int64_t T, int64_t K, int R, int RP,
                             float scale, float* out_f32, uint16_t* out_bf16, hipStream_t st) {
  dim3 grid((unsigned)((T + 15) / 16), (unsigned)(RP / 16));
  rowdot16_kernel<<<grid, 256, 0, st>>>((const uint16_t*)X, (const uint16_t*)Mt, T, K, R, RP, scale,
                                        out_f32, out_bf16);
  ARTK_CHECK_LAUNCH();
  return ARTK_OK;
}

}  // namespace artk

using namespace artk;

extern "C" {

size_t artk_lora_linear_fwd_workspace_bytes(int64_t T, int64_t in, int64_t out, int32_t r) {
  (void)in;
  (void)out;
  Workspace ws(nullptr, 0);
  ws.take<uint16_t>((size_t)T * round16(r));  // s * x A^T, bf16 [T,RP]
  return ws.used + 256;
}

int32_t artk_lora_linear_fwd(const void* x, const void* W, const void* A, const void* B, const void* bias,
                             float scale, int64_t T, int64_t in, int64_t out, int32_t r, void* y, float* xa,
                             void* workspace, size_t workspace_bytes, artk_stream_t stream) {
  int32_t rc = check_lora(T, in, out, r);
  if (rc) return rc;
  ARTK_CHECK_ARG(x && W && A && B && y && xa, "null pointer argument");
  ARTK_CHECK_ARG(aligned16(x) && aligned16(W) && aligned16(A) && aligned16(B) && aligned16(y),
                 "pointers must be 16-byte aligned");
  const int RP = round16(r);
  Workspace ws(workspace, workspace_bytes);
  uint16_t* xa16 = ws.take<uint16_t>((size_t)T * RP);
  if (!ws.ok()) {
    set_error("workspace too small: need %zu bytes, got %zu", ws.used, workspace_bytes);
    return ARTK_ERR_WORKSPACE_TOO_SMALL;
  }
  hipStream_t st = (hipStream_t)stream;
  if ((rc = launch_rowdot(x, A, T, in, r, RP, scale, xa, xa16, st))) return rc;
  return launch_lora_gemm(W, x, (const uint16_t*)B, xa16, (const uint16_t*)bias, y, out, T, in, r, RP, st);
}

// Scratch of the backward, carved in the same order by the size query and the call.
struct LoraBwdScratch {
  uint16_t *Bt, *At, *gb16;
  float *gb, *rowp_g, *colp_g, *colp_x, *dummy;
  StatsGeom gg, gx;
};
static void carve_lora_bwd(Workspace& ws, int64_t T, int64_t in, int64_t out, int r, LoraBwdScratch& c) {
  const int RP = round16(r);
  c.gg = stats_geom(T, out, r);
  c.gx = stats_geom(T, in, r);
  c.Bt = ws.take<uint16_t>((size_t)r * out);   // B^T [r,out]: factor of the g B product
  c.At = ws.take<uint16_t>((size_t)in * r);    // A^T [in,r]: low-rank factor of dx
  c.gb = ws.take<float>((size_t)T * r);        // g B, f32 [T,r]
  c.gb16 = ws.take<uint16_t>((size_t)T * RP);  // s * g B, bf16 [T,RP]
  c.rowp_g = ws.take<float>((size_t)c.gg.n_chunks * T * r);
  c.colp_g = ws.take<float>((size_t)c.gg.n_slabs * out * r);
  c.colp_x = ws.take<float>((size_t)c.gx.n_slabs * in * r);
  c.dummy = ws.take<float>(1024);
}

size_t artk_lora_linear_bwd_workspace_bytes(int64_t T, int64_t in, int64_t out, int32_t r) {
  Workspace ws(nullptr, 0);
  LoraBwdScratch c;
  carve_lora_bwd(ws, T, in, out, r, c);
  return ws.used + 256;
}

int32_t artk_lora_linear_bwd(const void* g, const void* x, const void* W_t, const void* A,
                             const void* B, const float* xa, float scale, int64_t T, int64_t in,
                             int64_t out, int32_t r, void* dx, float* dA, float* dB, void* workspace,
                             size_t workspace_bytes, artk_stream_t stream) {
  int32_t rc = check_lora(T, in, out, r);
  if (rc) return rc;
  ARTK_CHECK_ARG(g && x && W_t && A && B && xa && dx && dA && dB, "null pointer argument");
  ARTK_CHECK_ARG(aligned16(g) && aligned16(x) && aligned16(W_t) && aligned16(A) && aligned16(B) && aligned16(dx) && aligned16(xa) &&
                     aligned16(dA) && aligned16(dB),
                 "pointers must be 16-byte aligned");
  const int RP = round16(r);
  Workspace ws(workspace, workspace_bytes);
  LoraBwdScratch c;
  carve_lora_bwd(ws, T, in, out, r, c);
  if (!ws.ok()) {
    set_error("workspace too small: need %zu bytes, got %zu", ws.used, workspace_bytes);
    return ARTK_ERR_WORKSPACE_TOO_SMALL;
  }
  hipStream_t st = (hipStream_t)stream;
  if ((rc = launch_small_transpose2(B, c.Bt, 1, out, r, A, c.At, 1, r, in, st))) return rc;
  // one pass over g: partials of g B (over column chunks) and of g^T (x A^T) (over row slabs)
  if ((rc = launch_stats(g, T, out, c.Bt, xa, r, c.gg, c.rowp_g, c.colp_g, c.dummy, st))) return rc;
  {
    StatsReduceJob ja{c.rowp_g, c.gg.n_chunks, T, 1.f, c.gb, 0, c.gb16, RP, scale};
    StatsReduceJob jb{c.colp_g, c.gg.n_slabs, out, scale, dB, 0, nullptr, 0, 0.f};
    if ((rc = launch_stats_reduce(ja, jb, r, st))) return rc;
  }
  // dx = g W + (s g B) A
  if ((rc = launch_lora_gemm(W_t, g, c.At, c.gb16, nullptr, dx, in, T, out, r, RP, st))) return rc;
  // one pass over x: dA [r,in] = s (g B)^T x
  if ((rc = launch_stats(x, T, in, nullptr, c.gb, r, c.gx, nullptr, c.colp_x, c.dummy, st))) return rc;
  {
    StatsReduceJob ja{c.colp_x, c.gx.n_slabs, in, scale, dA, 1, nullptr, 0, 0.f};
    StatsReduceJob jb{nullptr, 0, 0, 0.f, nullptr, 0, nullptr, 0, 0.f};
    if ((rc = launch_stats_reduce(ja, jb, r, st))) return rc;
  }
  return ARTK_OK;
}

// ---- the same linear with the frozen weight kept as NF4 codes -------------------------------
// The bf16 weight exists only inside the call: it is dequantised into the workspace (forward:
// [out,in]; backward: [in,out], written transposed straight from the codes), consumed by the
// GEMM and forgotten, so neither a bf16 copy nor a transposed copy of W stays resident.
static int32_t check_nf4_weight(const artk_nf4_t* W, int64_t in) {
  ARTK_CHECK_ARG(W != nullptr && W->packed != nullptr, "null NF4 weight");
  ARTK_CHECK_ARG(W->blocksize >= 32 && in % W->blocksize == 0,
                 "the input size must be a multiple of the quantisation block size");
  return ARTK_OK;
}

size_t artk_lora_linear_fwd_nf4_workspace_bytes(int64_t T, int64_t in, int64_t out, int32_t r) {
  Workspace ws(nullptr, 0);
  ws.take<uint16_t>((size_t)out * in);
  ws.take<char>(artk_lora_linear_fwd_workspace_bytes(T, in, out, r));
  return ws.used + 256;
}

int32_t artk_lora_linear_fwd_nf4(const void* x, const artk_nf4_t* W, const void* A, const void* B,
                                 const void* bias, float scale, int64_t T, int64_t in, int64_t out, int32_t r,
                                 void* y, float* xa, void* workspace, size_t workspace_bytes,
                                 artk_stream_t stream) {
  int32_t rc = check_lora(T, in, out, r);
  if (rc) return rc;
  if ((rc = check_nf4_weight(W, in))) return rc;
  Workspace ws(workspace, workspace_bytes);
  uint16_t* Wd = ws.take<uint16_t>((size_t)out * in);
  const size_t inner = artk_lora_linear_fwd_workspace_bytes(T, in, out, r);
  char* rest = ws.take<char>(inner);
  if (!ws.ok()) {
    set_error("workspace too small: need %zu bytes, got %zu", ws.used, workspace_bytes);
    return ARTK_ERR_WORKSPACE_TOO_SMALL;
  }
  if ((rc = artk_nf4_dequant(W->packed, W->absmax, W->absmax_q, W->code2, W->absmax2, W->offset, out * in,
                             W->blocksize, Wd, stream)))
    return rc;
  return artk_lora_linear_fwd(x, Wd, A, B, bias, scale, T, in, out, r, y, xa, rest, inner, stream);
}

size_t artk_lora_linear_bwd_nf4_workspace_bytes(int64_t T, int64_t in, int64_t out, int32_t r) {
  Workspace ws(nullptr, 0);
  ws.take<uint16_t>((size_t)out * in);
  ws.take<char>(artk_lora_linear_bwd_workspace_bytes(T, in, out, r));
  return ws.used + 256;
}

int32_t artk_lora_linear_bwd_nf4(const void* g, const void* x, const artk_nf4_t* W, const void* A,
                                 const void* B, const float* xa, float scale, int64_t T, int64_t in,
                                 int64_t out, int32_t r, void* dx, float* dA, float* dB, void* workspace,
                                 size_t workspace_bytes, artk_stream_t stream) {
  int32_t rc = check_lora(T, in, out, r);
  if (rc) return rc;
  if ((rc = check_nf4_weight(W, in))) return rc;
  Workspace ws(workspace, workspace_bytes);
  uint16_t* Wt = ws.take<uint16_t>((size_t)out * in);
  const size_t inner = artk_lora_linear_bwd_workspace_bytes(T, in, out, r);
  char* rest = ws.take<char>(inner);
  if (!ws.ok()) {
    set_error("workspace too small: need %zu bytes, got %zu", ws.used, workspace_bytes);
    return ARTK_ERR_WORKSPACE_TOO_SMALL;
  }
  if ((rc = artk_nf4_dequant_t(W->packed, W->absmax, W->absmax_q, W->code2, W->absmax2, W->offset, out, in,
                               W->blocksize, Wt, stream)))
    return rc;
  return artk_lora_linear_bwd(g, x, Wt, A, B, xa, scale, T, in, out, r, dx, dA, dB, rest, inner, stream);
}

}  // extern "C"
