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
#include "gemm_plain8.hpp"
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

// Rank-r steps of one tile: acc += sum_e Qe[col, e] Pe[row, e].
__device__ __forceinline__ void lora_tile_lowrank(TileAcc<LORA_NI>& acc, const uint16_t* Pe, int r,
                                                  const uint16_t* Qe, int RP, int64_t M, int64_t N, int mt,
                                                  int nt) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int wm = wave_m<LORA_NI>(wave), wn = wave_n<LORA_NI>(wave);
  int64_t prow[4], qrow[LORA_NI];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    int64_t rr = (int64_t)mt * TILE + wm * 128 + i * 32 + (lane & 31);
    prow[i] = rr < M ? rr : M - 1;
  }
#pragma unroll
  for (int i = 0; i < LORA_NI; ++i) {
    int64_t c = (int64_t)nt * TILE + acc_col<LORA_NI>(wn, i, lane);
    qrow[i] = c < N ? c : N - 1;
  }
  lowrank_steps(acc, Pe, r, r, prow, Qe, RP, RP, qrow, RP);
}

// Optional bias and the bf16 store of one finished tile: out[col, m] (out is [N, M]).
__device__ __forceinline__ void lora_tile_store(TileAcc<LORA_NI>& acc, const uint16_t* bias, uint16_t* out,
                                                int64_t M, int64_t N, int mt, int nt) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int wm = wave_m<LORA_NI>(wave), wn = wave_n<LORA_NI>(wave);
  const int half = lane >> 5;
  if (bias != nullptr) {
    // element j of tile mi is output feature m0 + (j / 4) 8 + 4 half + j % 4
#pragma unroll
    for (int mi = 0; mi < 4; ++mi) {
      const int64_t m0 = (int64_t)mt * TILE + wm * 128 + mi * 32;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        int64_t mq = m0 + q * 8 + half * 4;
        mq = mq + 4 <= M ? mq : 0;  // rows past the end are never stored
        const bf16x4 bv = *(const bf16x4*)(bias + mq);
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
    const bool col_ok = col < N;
#pragma unroll
    for (int mi = 0; mi < 4; ++mi) {
      const int64_t m0 = (int64_t)mt * TILE + wm * 128 + mi * 32;
      if (m0 >= M) continue;  // wave-uniform
      if (m0 + 32 <= M) {
        if (col_ok) store_block_bf16(out + col * M + m0, acc.c[mi][ni], half);
      } else {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int64_t m = m0 + q * 8 + half * 4;
          if (m >= M || !col_ok) continue;
          bf16x4 o;
#pragma unroll
          for (int e = 0; e < 4; ++e) o[e] = (__bf16)acc.c[mi][ni][q * 4 + e];
          *(bf16x4*)(out + col * M + m) = o;
        }
      }
    }
  }
}

// Rank-r steps and bf16 store of one finished tile.
__device__ __forceinline__ void lora_gemm_epilogue(TileAcc<LORA_NI>& acc, const LoraGemmParams& p, int mt,
                                                   int nt) {
  if (p.Pe != nullptr) lora_tile_lowrank(acc, p.Pe, p.r, p.Qe, p.RP, p.M, p.N, mt, nt);
  lora_tile_store(acc, p.bias, p.out, p.M, p.N, mt, nt);
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
    PlainTileLoaders first;
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
      PlainTileLoaders cur;  // its first stage is already on the way
      cur.init(p.P, p.K, (int64_t)mt * TILE, p.M, p.Q, p.K, (int64_t)nt * TILE, p.N, 0, (int)p.K);
      gemm_tile_run_plain8<false>(acc, smem, cur);
    }
    if (more) {
      PlainTileLoaders nxt;
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
// Several products over one column operand in ONE persistent launch.
// A job is one output matrix out[n, m] (bf16 [N, M]); it sums one or more K segments,
//   out[n, m] = sum_s ( sum_k Q_s[n,k] P_s[m,k] + sum_e Qe_s[n,e] Pe_s[m,e] )  (+ bias[m]).
// Forward of projections that read the same x: one job per projection (P = W_i, Q = x), one
// segment each.  Input gradient of the same projections: one job (dx) whose segments are the
// projections (P = W_i^T [in, out_i], Q = g_i [T, out_i], K = out_i), so the upstream gradients
// are never concatenated and dx is written once.  A segment switch inside a tile costs one
// exposed first-stage fetch (the two LDS stages are busy until the segment's last K step).
// ----------------------------------------------------------------------------
constexpr int LORA_MAX_SEG = ARTK_LORA_MULTI_MAX;
struct LoraSeg {
  const void* P;       // [M,K] row operand
  const void* Q;       // [N,K] column operand
  const uint16_t* Pe;  // [M,r]
  const uint16_t* Qe;  // [N,RP]
  int64_t K;
  int r, RP;
};
struct LoraJob {
  uint16_t* out;         // [N,M]
  const uint16_t* bias;  // [M] or nullptr
  int64_t M;
  int MT, tile0, seg0, nseg;
};
struct LoraMultiParams {
  LoraSeg seg[LORA_MAX_SEG];
  LoraJob job[LORA_MAX_SEG];
  int64_t N;
  int NT, n_jobs, n_tiles;
};

__device__ __forceinline__ void lora_multi_locate(const LoraMultiParams& p, int t, int& j, int& mt, int& nt) {
  const int id = xcd_remap(t, p.n_tiles);
  j = 0;
  while (j + 1 < p.n_jobs && id >= p.job[j + 1].tile0) ++j;
  tile_coords(id - p.job[j].tile0, p.job[j].MT, p.NT, mt, nt);
}

__global__ __launch_bounds__(nthreads<LORA_NI>()) void lora_multi_gemm_kernel(LoraMultiParams p) {
  __shared__ __attribute__((aligned(1024))) char smem[GEMM_LDS_BYTES];
  int t = blockIdx.x;
  int j, mt, nt;
  lora_multi_locate(p, t, j, mt, nt);
  {
    const LoraSeg& sg = p.seg[p.job[j].seg0];
    PlainTileLoaders first;
    first.init(sg.P, sg.K, (int64_t)mt * TILE, p.job[j].M, sg.Q, sg.K, (int64_t)nt * TILE, p.N, 0, (int)sg.K);
    first.issue_first(smem);
  }
  for (;;) {
    const int t2 = t + gridDim.x;
    const bool more = t2 < p.n_tiles;
    int j2 = 0, mt2 = 0, nt2 = 0;
    if (more) lora_multi_locate(p, t2, j2, mt2, nt2);
    const int64_t M = p.job[j].M;
    const int seg0 = p.job[j].seg0, nseg = p.job[j].nseg;
    TileAcc<LORA_NI> acc;
    acc.zero();
    // (one branch around all segments, not one per segment: see gemm_plain8.hpp)
    if (plain8_leader()) {
      for (int s = 0; s < nseg; ++s) {
        const LoraSeg& sg = p.seg[seg0 + s];
        PlainTileLoaders cur;  // the first segment's first stage is already on the way
        cur.init(sg.P, sg.K, (int64_t)mt * TILE, M, sg.Q, sg.K, (int64_t)nt * TILE, p.N, 0, (int)sg.K);
        if (s > 0) cur.issue_first_leader(smem);
        gemm_tile_run<2, 2, false>(acc, smem, cur);
      }
    } else {
      for (int s = 0; s < nseg; ++s) {
        const NoLoaders none{0, (int)p.seg[seg0 + s].K};
        gemm_tile_run<2, 2, false>(acc, smem, none);
      }
    }
    if (more) {
      const LoraSeg& sg = p.seg[p.job[j2].seg0];
      PlainTileLoaders nxt;
      nxt.init(sg.P, sg.K, (int64_t)mt2 * TILE, p.job[j2].M, sg.Q, sg.K, (int64_t)nt2 * TILE, p.N, 0, (int)sg.K);
      nxt.issue_first(smem);
    }
    for (int s = 0; s < nseg; ++s) {
      const LoraSeg& sg = p.seg[seg0 + s];
      if (sg.Pe != nullptr) lora_tile_lowrank(acc, sg.Pe, sg.r, sg.Qe, sg.RP, M, p.N, mt, nt);
    }
    lora_tile_store(acc, p.job[j].bias, p.job[j].out, M, p.N, mt, nt);
    if (!more) break;
    t = t2;
    j = j2;
    mt = mt2;
    nt = nt2;
  }
}

// ----------------------------------------------------------------------------
// Row products: out[t, j] = sum_k X[t,k] Mt[j,k], Mt [R,K].  A block owns 16 rows
// of X and 16 rows j0..j0+15 of Mt (rows >= R read as zero); its 4 waves split K.
// Writes f32 [T,R] (unscaled) and bf16 [T,RP] (scaled, zero padded to RP).
// ----------------------------------------------------------------------------
__device__ __forceinline__ void rowdot16_body(const uint16_t* __restrict__ X, const uint16_t* __restrict__ Mt,
                                              int64_t T, int64_t K, int R, int RP, float scale,
                                              float* __restrict__ out_f32, uint16_t* __restrict__ out_bf16,
                                              int j0, floatx4 (*red)[64]) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int64_t t0 = (int64_t)blockIdx.x * 16;
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

__global__ __launch_bounds__(256) void rowdot16_kernel(const uint16_t* __restrict__ X,
                                                       const uint16_t* __restrict__ Mt, int64_t T,
                                                       int64_t K, int R, int RP, float scale,
                                                       float* __restrict__ out_f32,
                                                       uint16_t* __restrict__ out_bf16) {
  __shared__ floatx4 red[3][64];
  rowdot16_body(X, Mt, T, K, R, RP, scale, out_f32, out_bf16, blockIdx.y * 16, red);
}

// The same for several factors over one X in one launch: blockIdx.y walks the 16-row groups of
// factor 0, then of factor 1, ...; each factor has its own outputs.
struct RowdotMulti {
  const uint16_t* Mt[LORA_MAX_SEG];
  float* out_f32[LORA_MAX_SEG];
  uint16_t* out_bf16[LORA_MAX_SEG];
  int R[LORA_MAX_SEG], RP[LORA_MAX_SEG], y0[LORA_MAX_SEG + 1];
  int n;
};
__global__ __launch_bounds__(256) void rowdot16_multi_kernel(const uint16_t* __restrict__ X, RowdotMulti m,
                                                             int64_t T, int64_t K, float scale) {
  __shared__ floatx4 red[3][64];
  const int by = blockIdx.y;
  int i = 0;
  while (i + 1 < m.n && by >= m.y0[i + 1]) ++i;
  rowdot16_body(X, m.Mt[i], T, K, m.R[i], m.RP[i], scale, m.out_f32[i], m.out_bf16[i], (by - m.y0[i]) * 16, red);
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
  ARTK_CHECK_ARG(aligned16(x) && aligned16(W) && aligned16(A) && aligned16(B) && aligned16(y) &&
                     (bias == nullptr || aligned16(bias)),
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

// ---- several projections of the same input -------------------------------------------------
static int32_t check_multi(const artk_lora_proj_t* proj, int32_t n, int64_t T, int64_t in, bool bwd) {
  ARTK_CHECK_ARG(proj != nullptr && n >= 1 && n <= ARTK_LORA_MULTI_MAX, "1 to %d projections", ARTK_LORA_MULTI_MAX);
  int r_total = 0;
  for (int i = 0; i < n; ++i) {
    const artk_lora_proj_t& q = proj[i];
    int32_t rc = check_lora(T, in, q.out, q.r);
    if (rc) return rc;
    r_total += q.r;
    if (bwd) {
      ARTK_CHECK_ARG(q.W_t && q.A && q.B && q.g && q.xa && q.dA && q.dB, "projection %d: null pointer argument", i);
      ARTK_CHECK_ARG(aligned16(q.W_t) && aligned16(q.A) && aligned16(q.B) && aligned16(q.g) && aligned16(q.xa) &&
                         aligned16(q.dA) && aligned16(q.dB),
                     "projection %d: pointers must be 16-byte aligned", i);
    } else {
      ARTK_CHECK_ARG(q.W && q.A && q.B && q.y && q.xa, "projection %d: null pointer argument", i);
      ARTK_CHECK_ARG(aligned16(q.W) && aligned16(q.A) && aligned16(q.B) && aligned16(q.y) && aligned16(q.xa) &&
                         (q.bias == nullptr || aligned16(q.bias)),
                     "projection %d: pointers must be 16-byte aligned", i);
    }
  }
  if (bwd && r_total > 64) {
    set_error("the ranks of the projections add up to %d; at most 64 in one call", r_total);
    return ARTK_ERR_UNSUPPORTED_SHAPE;
  }
  return ARTK_OK;
}

static int lora_num_cus() {
  int cus = 0, dev = 0;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
    cus = 256;
  return cus;
}

static int32_t launch_lora_multi(const LoraMultiParams& p, hipStream_t st) {
  prof_begin(PROF_LORA_GEMM, st);
  const int cus = lora_num_cus();
  lora_multi_gemm_kernel<<<(unsigned)(p.n_tiles < cus ? p.n_tiles : cus), nthreads<LORA_NI>(), 0, st>>>(p);
  prof_end(PROF_LORA_GEMM, st);
  ARTK_CHECK_LAUNCH();
  return ARTK_OK;
}

size_t artk_lora_linear_multi_fwd_workspace_bytes(int64_t T, int64_t in, const artk_lora_proj_t* proj,
                                                  int32_t n) {
  (void)in;
  Workspace ws(nullptr, 0);
  for (int i = 0; proj != nullptr && i < n && i < ARTK_LORA_MULTI_MAX; ++i)
    ws.take<uint16_t>((size_t)T * round16(proj[i].r));
  return ws.used + 256;
}

int32_t artk_lora_linear_multi_fwd(const void* x, const artk_lora_proj_t* proj, int32_t n, float scale,
                                   int64_t T, int64_t in, void* workspace, size_t workspace_bytes,
                                   artk_stream_t stream) {
  int32_t rc = check_multi(proj, n, T, in, false);
  if (rc) return rc;
  ARTK_CHECK_ARG(x != nullptr && aligned16(x), "x must be a 16-byte aligned pointer");
  Workspace ws(workspace, workspace_bytes);
  uint16_t* xa16[ARTK_LORA_MULTI_MAX];
  for (int i = 0; i < n; ++i) xa16[i] = ws.take<uint16_t>((size_t)T * round16(proj[i].r));
  if (!ws.ok()) {
    set_error("workspace too small: need %zu bytes, got %zu", ws.used, workspace_bytes);
    return ARTK_ERR_WORKSPACE_TOO_SMALL;
  }
  hipStream_t st = (hipStream_t)stream;
  RowdotMulti m;
  LoraMultiParams p;
  m.n = n;
  int y = 0, tile = 0;
  p.N = T;
  p.NT = (int)((T + TILE - 1) / TILE);
  p.n_jobs = n;
  for (int i = 0; i < n; ++i) {
    const artk_lora_proj_t& q = proj[i];
    const int RP = round16(q.r);
    m.Mt[i] = (const uint16_t*)q.A;
    m.out_f32[i] = q.xa;
    m.out_bf16[i] = xa16[i];
    m.R[i] = q.r;
    m.RP[i] = RP;
    m.y0[i] = y;
    y += RP / 16;
    p.seg[i] = LoraSeg{q.W, x, (const uint16_t*)q.B, xa16[i], in, q.r, RP};
    const int MT = (int)((q.out + TILE - 1) / TILE);
    p.job[i] = LoraJob{(uint16_t*)q.y, (const uint16_t*)q.bias, q.out, MT, tile, i, 1};
    tile += MT * p.NT;
  }
  m.y0[n] = y;
  p.n_tiles = tile;
  dim3 grid((unsigned)((T + 15) / 16), (unsigned)y);
  rowdot16_multi_kernel<<<grid, 256, 0, st>>>((const uint16_t*)x, m, T, in, scale);
  ARTK_CHECK_LAUNCH();
  return launch_lora_multi(p, st);
}

struct LoraMultiBwdScratch {
  LoraBwdScratch one[ARTK_LORA_MULTI_MAX];  // per projection: Bt, At, gb16, rowp_g, colp_g (gb, colp_x unused)
  float* gb_cat;   // [T, r_total]: g_i B_i side by side, the Y of the pass over x
  float* colp_x;   // [n_slabs][in][r_total]
  float* dummy;
  StatsGeom gx;
  int r_total;
};
static void carve_lora_multi_bwd(Workspace& ws, int64_t T, int64_t in, const artk_lora_proj_t* proj, int n,
                                 LoraMultiBwdScratch& c) {
  c.r_total = 0;
  for (int i = 0; i < n; ++i) c.r_total += proj[i].r;
  for (int i = 0; i < n; ++i) {
    const int64_t out = proj[i].out;
    const int r = proj[i].r, RP = round16(r);
    LoraBwdScratch& o = c.one[i];
    o.gg = stats_geom(T, out, r);
    o.Bt = ws.take<uint16_t>((size_t)r * out);
    o.At = ws.take<uint16_t>((size_t)in * r);
    o.gb16 = ws.take<uint16_t>((size_t)T * RP);
    o.rowp_g = ws.take<float>((size_t)o.gg.n_chunks * T * r);
    o.colp_g = ws.take<float>((size_t)o.gg.n_slabs * out * r);
  }
  c.gx = stats_geom(T, in, c.r_total);
  c.gb_cat = ws.take<float>((size_t)T * c.r_total);
  c.colp_x = ws.take<float>((size_t)c.gx.n_slabs * in * c.r_total);
  c.dummy = ws.take<float>(1024);
}

size_t artk_lora_linear_multi_bwd_workspace_bytes(int64_t T, int64_t in, const artk_lora_proj_t* proj,
                                                  int32_t n) {
  if (proj == nullptr || n < 1 || n > ARTK_LORA_MULTI_MAX) return 0;
  Workspace ws(nullptr, 0);
  LoraMultiBwdScratch c;
  carve_lora_multi_bwd(ws, T, in, proj, n, c);
  return ws.used + 256;
}

int32_t artk_lora_linear_multi_bwd(const void* x, const artk_lora_proj_t* proj, int32_t n, float scale,
                                   int64_t T, int64_t in, void* dx, void* workspace, size_t workspace_bytes,
                                   artk_stream_t stream) {
  int32_t rc = check_multi(proj, n, T, in, true);
  if (rc) return rc;
  ARTK_CHECK_ARG(x != nullptr && dx != nullptr && aligned16(x) && aligned16(dx),
                 "x and dx must be 16-byte aligned pointers");
  Workspace ws(workspace, workspace_bytes);
  LoraMultiBwdScratch c;
  carve_lora_multi_bwd(ws, T, in, proj, n, c);
  if (!ws.ok()) {
    set_error("workspace too small: need %zu bytes, got %zu", ws.used, workspace_bytes);
    return ARTK_ERR_WORKSPACE_TOO_SMALL;
  }
  hipStream_t st = (hipStream_t)stream;
  LoraMultiParams p;
  p.N = T;
  p.NT = (int)((T + TILE - 1) / TILE);
  p.n_jobs = 1;
  const int MT = (int)((in + TILE - 1) / TILE);
  p.job[0] = LoraJob{(uint16_t*)dx, nullptr, in, MT, 0, 0, n};
  p.n_tiles = MT * p.NT;
  StatsReduceJob jx{c.colp_x, c.gx.n_slabs, in, scale, nullptr, 1, nullptr, 0, 0.f};
  jx.n_split = n;
  SmallTransposeMulti tr;
  StatsMulti sm;
  StatsReduceMulti rm;
  tr.n = 2 * n;
  sm.n = n;
  rm.n = 2 * n;
  bool any_wide = false, any_narrow = false;
  int r0 = 0;
  for (int i = 0; i < n; ++i) {
    const artk_lora_proj_t& q = proj[i];
    LoraBwdScratch& o = c.one[i];
    const int RP = round16(q.r);
    (q.r > 32 ? any_wide : any_narrow) = true;
    tr.t[2 * i] = SmallTranspose{(const uint16_t*)q.B, o.Bt, 1, q.out, q.r};
    tr.t[2 * i + 1] = SmallTranspose{(const uint16_t*)q.A, o.At, 1, q.r, in};
    // one pass over g_i: partials of g_i B_i (over column chunks) and of g_i^T (x A_i^T) (over row slabs)
    sm.p[i] = stats_params(q.g, T, q.out, o.Bt, q.xa, q.r, o.gg, o.rowp_g, o.colp_g, c.dummy);
    StatsReduceJob ja{o.rowp_g, o.gg.n_chunks, T, 1.f, c.gb_cat, 0, o.gb16, RP, scale};
    ja.out_ld = c.r_total;
    ja.out_off = r0;
    rm.job[2 * i] = ja;
    rm.job[2 * i + 1] = StatsReduceJob{o.colp_g, o.gg.n_slabs, q.out, scale, q.dB, 0, nullptr, 0, 0.f};
    rm.R[2 * i] = rm.R[2 * i + 1] = q.r;
    p.seg[i] = LoraSeg{q.W_t, q.g, o.At, o.gb16, q.out, q.r, RP};
    jx.outs[i] = q.dA;
    jx.e_start[i] = r0;
    r0 += q.r;
  }
  jx.e_start[n] = r0;
  if ((rc = launch_small_transpose_multi(tr, st))) return rc;
  if (any_wide && any_narrow) {  // the stats kernel has one shape per side of rank 32: one launch per projection
    for (int i = 0; i < n; ++i) {
      const StatsParams& sp = sm.p[i];
      if (sp.R > 32)
        lora_stats_kernel<2, 2, 2, false><<<(unsigned)(sp.n_slabs * sp.n_chunks), 256, 0, st>>>(sp);
      else
        lora_stats_kernel<1, 4, 3, false><<<(unsigned)(sp.n_slabs * sp.n_chunks), 256, 0, st>>>(sp);
      ARTK_CHECK_LAUNCH();
    }
  } else if ((rc = launch_stats_multi(sm, any_wide, st))) {
    return rc;
  }
  if ((rc = launch_stats_reduce_multi(rm, st))) return rc;
  // dx = sum_i ( g_i W_i + (s g_i B_i) A_i ): one launch, the projections as K segments
  if ((rc = launch_lora_multi(p, st))) return rc;
  // one pass over x: [dA_0; dA_1; ...] = s [g_0 B_0 | g_1 B_1 | ...]^T x
  if ((rc = launch_stats(x, T, in, nullptr, c.gb_cat, c.r_total, c.gx, nullptr, c.colp_x, c.dummy, st))) return rc;
  StatsReduceJob none{nullptr, 0, 0, 0.f, nullptr, 0, nullptr, 0, 0.f};
  return launch_stats_reduce(jx, none, c.r_total, st);
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
