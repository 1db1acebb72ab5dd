// MoE expert path for gfx950: router top-k, stable expert-contiguous
// permutation, and per-expert LoRA linears as grouped GEMMs
//   y[i,:] = x[row(i),:] W_e^T + s (x[row(i),:] A_e^T) B_e^T      e = expert of row i
// over the permuted (token, expert) rows, with their backward.
//
// The reference has no MoE code at this commit; the contract comes from the
// benchmark configuration (128 experts, top-8, Qwen3-30B-A3B-style expert
// shapes, rank-8 LoRA per expert).  Routing follows the usual definition
// (softmax over router logits in fp32, top-k, renormalise); the selection is
// made on the logits, which order like the softmax, ties to the lower expert
// index, and the permutation is the stable sort of the token-major (token, slot)
// list by expert id, so both integer outputs are reproducible bit for bit.
#include "common.hpp"
#include "gemm_nt.hpp"
#include "lora_common.hpp"
#include "skinny_stats.hpp"

#include <math.h>

namespace artk {

// ----------------------------------------------------------------------------
// Routing: one wavefront per token.
// ----------------------------------------------------------------------------
constexpr int MOE_NI = 2;  // 8 waves, 2 per SIMD (see gemm_nt.hpp)
constexpr int MOE_MAX_E = 256;
constexpr int MOE_MAX_K = 16;

__global__ __launch_bounds__(256) void moe_topk_kernel(const float* __restrict__ logits, int64_t T,
                                                       int E, int k, int* __restrict__ topk_idx,
                                                       float* __restrict__ topk_w) {
  const int lane = threadIdx.x & 63;
  const int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (t >= T) return;
  // NaN counts as -inf, so the order below is total: decreasing value, ties (also
  // among -inf) to the lower expert index; every round picks an index in [0, E).
  float x[4];
  unsigned taken = 0;  // bit i: element i of this lane is selected or past E
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int e = lane + 64 * i;
    float v = e < E ? logits[t * E + e] : -INFINITY;
    x[i] = v == v ? v : -INFINITY;
    if (e >= E) taken |= 1u << i;
  }
  float m = fmaxf(fmaxf(x[0], x[1]), fmaxf(x[2], x[3]));
  m = wave_max(m);
  float myp = 0.f;  // lane j keeps the probability mass of slot j
  float psum = 0.f;
  for (int j = 0; j < k; ++j) {
    float bv = -INFINITY;
    int bi = 0x7fffffff;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (!(taken >> i & 1) && (bi == 0x7fffffff || x[i] > bv)) {
        bv = x[i];
        bi = lane + 64 * i;
      }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(bv, o, 64);
      const int oi = __shfl_xor(bi, o, 64);
      if (oi != 0x7fffffff && (bi == 0x7fffffff || ov > bv || (ov == bv && oi < bi))) {
        bv = ov;
        bi = oi;
      }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (lane + 64 * i == bi) taken |= 1u << i;
    // exp(-inf - m) = 0; a row without any finite logit (m = -inf) has no mass at all
    const float pj = bv == -INFINITY ? 0.f : expf(bv - m);
    psum += pj;
    if (lane == j) myp = pj;
    if (lane == 0) topk_idx[t * k + j] = bi;
  }
  if (lane < k) topk_w[t * k + lane] = psum > 0.f ? myp / psum : 0.f;
}

// ----------------------------------------------------------------------------
// Stable counting sort of the n = T*k keys (expert ids) in chunks of 1024.
// ----------------------------------------------------------------------------
constexpr int PERM_CHUNK = 1024;

__global__ __launch_bounds__(PERM_CHUNK) void moe_hist_kernel(const int* __restrict__ keys, int n,
                                                              int E, int* __restrict__ cnt) {
  __shared__ int hist[MOE_MAX_E];
  for (int i = threadIdx.x; i < E; i += PERM_CHUNK) hist[i] = 0;
  __syncthreads();
  const int f = blockIdx.x * PERM_CHUNK + threadIdx.x;
  // keys come from moe_topk_kernel and lie in [0, E); anything else is ignored
  if (f < n && (unsigned)keys[f] < (unsigned)E) atomicAdd(&hist[keys[f]], 1);
  __syncthreads();
  for (int i = threadIdx.x; i < E; i += PERM_CHUNK) cnt[blockIdx.x * E + i] = hist[i];
}

// offsets[e]: first sorted position of expert e; base[b][e]: first sorted
// position of chunk b's entries of expert e; tile_prefix / blk_prefix: prefix
// sums of ceil(rows_e / 256) and ceil(rows_e / 16) (work lists of the grouped
// kernels).  One block of 1024 threads: thread (part, e) walks a quarter of the
// chunks of expert e, eight independent loads at a time.
constexpr int SCAN_PARTS = 4;
__global__ __launch_bounds__(SCAN_PARTS * MOE_MAX_E) void moe_scan_kernel(const int* __restrict__ cnt, int nb, int E,
                                                                          int* __restrict__ offsets,
                                                                          int* __restrict__ base,
                                                                          int* __restrict__ tile_prefix,
                                                                          int* __restrict__ blk_prefix) {
  __shared__ int part[SCAN_PARTS][MOE_MAX_E];
  __shared__ int wsum[3][MOE_MAX_E / 64];
  __shared__ int off[MOE_MAX_E];
  const int e = threadIdx.x % MOE_MAX_E, pt = threadIdx.x / MOE_MAX_E;
  const int per = (nb + SCAN_PARTS - 1) / SCAN_PARTS;
  const int b0 = pt * per, b1 = b0 + per < nb ? b0 + per : nb;
  int s = 0;
  if (e < E) {
    for (int b = b0; b < b1; b += 8) {
      int v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = b + u < b1 ? cnt[(b + u) * E + e] : 0;
#pragma unroll
      for (int u = 0; u < 8; ++u) s += v[u];
    }
  }
  part[pt][e] = s;
  __syncthreads();
  // exclusive prefix sums over the experts (threads of part 0: one expert each)
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int tot = 0, run = 0, tp = 0, bp = 0;
  if (pt == 0) {
    if (e < E)
#pragma unroll
      for (int q = 0; q < SCAN_PARTS; ++q) tot += part[q][e];
    run = tot;
    tp = (tot + TILE - 1) / TILE;
    bp = (tot + 15) / 16;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const int a = __shfl_up(run, d, 64), t = __shfl_up(tp, d, 64), c = __shfl_up(bp, d, 64);
      if (lane >= d) {
        run += a;
        tp += t;
        bp += c;
      }
    }
    if (lane == 63) {
      wsum[0][wave] = run;
      wsum[1][wave] = tp;
      wsum[2][wave] = bp;
    }
  }
  __syncthreads();
  if (pt == 0) {
    for (int w = 0; w < wave; ++w) {
      run += wsum[0][w];
      tp += wsum[1][w];
      bp += wsum[2][w];
    }
    // inclusive sums -> entry e + 1; entry 0 is zero
    if (e < E) {
      offsets[e + 1] = run;
      tile_prefix[e + 1] = tp;
      blk_prefix[e + 1] = bp;
      off[e] = run - tot;
    }
    if (e == 0) {
      offsets[0] = 0;
      tile_prefix[0] = 0;
      blk_prefix[0] = 0;
    }
  }
  __syncthreads();
  if (e < E) {
    int pos = off[e];
    for (int q = 0; q < pt; ++q) pos += part[q][e];
    for (int b = b0; b < b1; b += 8) {
      int v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = b + u < b1 ? cnt[(b + u) * E + e] : 0;
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        if (b + u < b1) base[(b + u) * E + e] = pos;
        pos += v[u];
      }
    }
  }
}

// Stable placement of one chunk: position = base[chunk][key] + number of earlier
// entries of the chunk with the same key.  That rank is the count in the earlier
// waves (per-wave histograms in LDS) plus the count among the earlier lanes of the
// own wave (64 shuffles), instead of a scan over the whole chunk per thread.
__global__ __launch_bounds__(PERM_CHUNK) void moe_scatter_kernel(const int* __restrict__ keys, int n,
                                                                 int E, int k,
                                                                 const int* __restrict__ base,
                                                                 int* __restrict__ perm,
                                                                 int* __restrict__ inv_perm,
                                                                 int* __restrict__ row_token) {
  constexpr int NW = PERM_CHUNK / 64;
  __shared__ int hist[NW][256];  // E <= 256
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int i = threadIdx.x; i < NW * 256; i += PERM_CHUNK) (&hist[0][0])[i] = 0;
  __syncthreads();
  const int f = blockIdx.x * PERM_CHUNK + threadIdx.x;
  int key = f < n ? keys[f] : -1;
  if ((unsigned)key >= (unsigned)E) key = -1;  // never produced by moe_topk_kernel
  if (key >= 0) atomicAdd(&hist[wave][key], 1);
  int rank = 0;
  for (int j = 0; j < 64; ++j) {
    const int kj = __shfl(key, j, 64);
    rank += (j < lane && kj == key) ? 1 : 0;
  }
  __syncthreads();
  if (key >= 0) {
    for (int w = 0; w < wave; ++w) rank += hist[w][key];
    const int pos = base[blockIdx.x * E + key] + rank;
    perm[pos] = f;
    inv_perm[f] = pos;
    row_token[pos] = f / k;
  }
}

// Largest g with prefix[g] <= x, for a non-decreasing prefix[0..G] with prefix[G] > x.
__device__ __forceinline__ int find_group(const int* __restrict__ prefix, int G, int x) {
  int lo = 0, hi = G;
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (prefix[mid] <= x) lo = mid; else hi = mid;
  }
  return lo;
}

// ----------------------------------------------------------------------------
// Grouped GEMM: 256-row tiles never straddle experts.
// ----------------------------------------------------------------------------
struct MoeGemmParams {
  const void* W;           // [E,M,K] bf16
  const void* X;           // activations, [*,K] bf16
  const int* gather;       // permuted row i reads X row gather[i]; nullptr: row i
  const uint16_t* Pe;      // [E,M,r] low-rank factor of the weights
  const uint16_t* Qe;      // [n_rows,RP] zero-padded, scaled low-rank activations
  uint16_t* out;           // [n_rows,M]
  const int* offsets;      // [E+1]
  const int* tile_prefix;  // [E+1]
  int64_t M, K;
  int E, r, RP, MT;
};

// One tile of the grouped product: expert, rows and weight tile.
struct MoeTile {
  int e, mt, nvalid;
  int64_t row0, row_end;
};

__device__ __forceinline__ MoeTile moe_tile(const MoeGemmParams& p, int t, int n_work) {
  // Ids run expert by expert and, inside an expert, weight tile by weight tile over its row
  // tiles: the two or three work-groups that need the same weight tile have neighbouring ids,
  // start together and read it from HBM once (the L2 of their XCD serves the others); the MT
  // work-groups that share a row tile are only a few ids apart and still run side by side.
  const int id = xcd_remap(t, n_work);
  MoeTile m;
  m.e = find_group(p.tile_prefix, p.E, id / p.MT);
  const int first = p.tile_prefix[m.e], n_e = p.tile_prefix[m.e + 1] - first;
  const int local = id - first * p.MT;
  m.mt = local / n_e;
  m.row0 = p.offsets[m.e] + (int64_t)(local - m.mt * n_e) * TILE;
  m.row_end = p.offsets[m.e + 1];
  m.nvalid = (int)(m.row_end - m.row0 < TILE ? m.row_end - m.row0 : TILE);
  return m;
}

__device__ __forceinline__ void moe_tile_loaders(TileLoaders<MOE_NI>& L, const MoeGemmParams& p,
                                                 const MoeTile& m) {
  // rows past the expert's end are not fetched (their output columns are never stored)
  L.init((const char*)p.W + (int64_t)m.e * p.M * p.K * 2, p.K, (int64_t)m.mt * TILE, p.M, p.X, p.K, m.row0,
         m.row_end, 0, (int)p.K, p.gather, true);
}

// Persistent work-groups: tiles t, t + grid, ... of the device-side work list; the
// next tile's first DMA stage starts before the rank-r steps and the store of the
// current one (short K loops: 12 or 32 steps per tile).
__global__ __launch_bounds__(nthreads<MOE_NI>()) void moe_gemm_kernel(MoeGemmParams p) {
  __shared__ __attribute__((aligned(1024))) char smem[GEMM_LDS_BYTES];
  const int n_work = p.tile_prefix[p.E] * p.MT;
  int t = blockIdx.x;
  if (t >= n_work) return;
  MoeTile cur = moe_tile(p, t, n_work);
  {
    TileLoaders<MOE_NI> first;
    moe_tile_loaders(first, p, cur);
    first.issue_first(smem);
  }
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int wm = wave_m<MOE_NI>(wave), wn = wave_n<MOE_NI>(wave);
  const int half = lane >> 5;
  for (;;) {
    const int t2 = t + gridDim.x;
    const bool more = t2 < n_work;
    MoeTile nxt = cur;
    if (more) nxt = moe_tile(p, t2, n_work);

    TileAcc<MOE_NI> acc;
    acc.zero();
    {
      TileLoaders<MOE_NI> L;  // its first stage is already on the way
      moe_tile_loaders(L, p, cur);
      gemm_tile_run_cols(acc, smem, L, cur.nvalid);  // a tail tile computes only its live 32-row blocks
    }
    if (more) {
      TileLoaders<MOE_NI> L;
      moe_tile_loaders(L, p, nxt);
      L.issue_first(smem);
    }

    const int e = cur.e, mt = cur.mt, nvalid = cur.nvalid;
    const int64_t row0 = cur.row0;
    if (p.Pe != nullptr) {
      int64_t prow[4], qrow[MOE_NI];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        int64_t r = (int64_t)mt * TILE + wm * 128 + i * 32 + (lane & 31);
        prow[i] = r < p.M ? r : p.M - 1;
      }
#pragma unroll
      for (int i = 0; i < MOE_NI; ++i) {
        int c = acc_col<MOE_NI>(wn, i, lane);
        qrow[i] = row0 + (c < nvalid ? c : nvalid - 1);
      }
      lowrank_steps(acc, p.Pe + (int64_t)e * p.M * p.r, p.r, p.r, prow, p.Qe, p.RP, p.RP, qrow, p.RP);
    }

#pragma unroll
    for (int ni = 0; ni < MOE_NI; ++ni) {
      // lanes l and l + 32 share the column, so they take these branches together
      // (store_block_bf16 exchanges data between them)
      const int c = acc_col<MOE_NI>(wn, ni, lane);
      const bool col_ok = c < nvalid;
#pragma unroll
      for (int mi = 0; mi < 4; ++mi) {
        const int64_t m0 = (int64_t)mt * TILE + wm * 128 + mi * 32;
        if (m0 >= p.M) continue;  // wave-uniform
        if (m0 + 32 <= p.M) {
          if (col_ok) store_block_bf16(p.out + (row0 + c) * p.M + m0, acc.c[mi][ni], half);
        } else {
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const int64_t m = m0 + q * 8 + half * 4;
            if (m >= p.M || !col_ok) continue;
            bf16x4 o;
#pragma unroll
            for (int k = 0; k < 4; ++k) o[k] = (__bf16)acc.c[mi][ni][q * 4 + k];
            *(bf16x4*)(p.out + (row0 + c) * p.M + m) = o;
          }
        }
      }
    }
    if (!more) break;
    t = t2;
    cur = nxt;
  }
}

// Grouped row products: 16-row blocks never straddle experts.
//   out[i, j] = sum_k X[row(i), k] Mt_e[j, k],  Mt [E,R,K]
__global__ __launch_bounds__(256) void moe_rowdot16_kernel(
    const uint16_t* __restrict__ X, const int* __restrict__ gather, const uint16_t* __restrict__ Mt,
    const int* __restrict__ offsets, const int* __restrict__ blk_prefix, int E, int64_t K, int R,
    int RP, float scale, float* __restrict__ out_f32, uint16_t* __restrict__ out_bf16) {
  __shared__ floatx4 red[3][64];
  const int b = blockIdx.x;
  if (b >= blk_prefix[E]) return;
  const int e = find_group(blk_prefix, E, b);
  const int64_t row0 = offsets[e] + (int64_t)(b - blk_prefix[e]) * 16;
  const int64_t row_end = offsets[e + 1];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int jm = blockIdx.y * 16 + (lane & 15);
  int64_t row = row0 + (lane & 15);
  if (row >= row_end) row = row_end - 1;
  const int64_t src = gather ? gather[row] : row;
  const uint16_t* xp = X + src * K + (lane >> 4) * 8;
  const uint16_t* mp = Mt + ((int64_t)e * R + (jm < R ? jm : 0)) * K + (lane >> 4) * 8;
  floatx4 acc = rowdot_accumulate(xp, mp, jm < R, K, wave);
  acc = rowdot_block_sum(acc, red);
  if (wave == 0) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int64_t i = row0 + (lane >> 4) * 4 + q;
      if (i < row_end) {
        if (jm < R) out_f32[i * R + jm] = acc[q];
        out_bf16[i * RP + jm] = f32_to_bf16(acc[q] * scale);
      }
    }
  }
}

__global__ __launch_bounds__(256) void transpose_bf16_batched_kernel(const uint16_t* __restrict__ in,
                                                                     uint16_t* __restrict__ out,
                                                                     int64_t R, int64_t C) {
  __shared__ uint16_t tile[64][66];
  in += (int64_t)blockIdx.z * R * C;
  out += (int64_t)blockIdx.z * R * C;
  const int64_t r0 = (int64_t)blockIdx.y * 64, c0 = (int64_t)blockIdx.x * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int i = ty; i < 64; i += 4) {
    int64_t r = r0 + i, c = c0 + tx;
    tile[i][tx] = (r < R && c < C) ? in[r * C + c] : (uint16_t)0;
  }
  __syncthreads();
  for (int i = ty; i < 64; i += 4) {
    int64_t c = c0 + i, r = r0 + tx;
    if (c < C && r < R) out[c * R + r] = tile[tx][i];
  }
}

static int32_t check_moe(int64_t n_rows, int64_t in, int64_t out, int E, int r) {
  ARTK_CHECK_ARG(n_rows > 0 && in > 0 && out > 0 && E > 0 && r > 0, "sizes must be positive");
  if (in % BK != 0 || out % BK != 0) {
    set_error("in (%lld) and out (%lld) must be multiples of %d", (long long)in, (long long)out, BK);
    return ARTK_ERR_UNSUPPORTED_SHAPE;
  }
  if (r % 8 != 0 || r > 64 || E > MOE_MAX_E) {
    set_error("LoRA rank must be a multiple of 8 and <= 64, experts <= %d", MOE_MAX_E);
    return ARTK_ERR_UNSUPPORTED_SHAPE;
  }
  if (n_rows >= (1ll << 31) / 8) {
    set_error("too many rows");
    return ARTK_ERR_UNSUPPORTED_SHAPE;
  }
  return ARTK_OK;
}

static int32_t launch_moe_gemm(const void* W, const void* X, const int* gather, const uint16_t* Pe,
                               const uint16_t* Qe, void* out, const int* offsets,
                               const int* tile_prefix, int64_t n_rows, int64_t M, int64_t K, int E,
                               int r, int RP, hipStream_t st) {
  MoeGemmParams p;
  p.W = W;
  p.X = X;
  p.gather = gather;
  p.Pe = Pe;
  p.Qe = Qe;
  p.out = (uint16_t*)out;
  p.offsets = offsets;
  p.tile_prefix = tile_prefix;
  p.M = M;
  p.K = K;
  p.E = E;
  p.r = r;
  p.RP = RP;
  p.MT = (int)((M + TILE - 1) / TILE);
  const int64_t max_row_tiles = (n_rows + TILE - 1) / TILE + E;
  prof_begin(PROF_MOE_GEMM, st);
  {
    // persistent: one work-group per CU walks the device-side work list
    int cus = 0, dev = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
      cus = 256;
    const int64_t upper = (int64_t)max_row_tiles * p.MT;
    moe_gemm_kernel<<<(unsigned)(upper < cus ? upper : cus), nthreads<MOE_NI>(), 0, st>>>(p);
  }
  prof_end(PROF_MOE_GEMM, st);
  ARTK_CHECK_LAUNCH();
  return ARTK_OK;
}

static int32_t launch_moe_rowdot(const void* X, const int* gather, const uint16_t* Mt,
                                 const int* offsets, const int* blk_prefix, int64_t n_rows, int E,
                                 int64_t K, int R, int RP, float scale, float* out_f32,
                                 uint16_t* out_bf16, hipStream_t st) {
  dim3 grid((unsigned)((n_rows + 15) / 16 + E), (unsigned)(RP / 16));
  moe_rowdot16_kernel<<<grid, 256, 0, st>>>((const uint16_t*)X, gather, Mt, offsets, blk_prefix, E, K,
                                            R, RP, scale, out_f32, out_bf16);
  ARTK_CHECK_LAUNCH();
  return ARTK_OK;
}

}  // namespace artk

using namespace artk;

extern "C" {

size_t artk_moe_route_workspace_bytes(int64_t T, int32_t E, int32_t k) {
  Workspace ws(nullptr, 0);
  const int64_t n = T * k;
  const int64_t nb = (n + PERM_CHUNK - 1) / PERM_CHUNK;
  ws.take<int>((size_t)(nb * E));
  ws.take<int>((size_t)(nb * E));
  return ws.used + 256;
}

int32_t artk_moe_route(const float* router_logits, int64_t T, int32_t E, int32_t k, int32_t* topk_idx,
                       float* topk_w, int32_t* perm, int32_t* inv_perm, int32_t* row_token,
                       int32_t* expert_offsets, int32_t* tile_prefix, int32_t* blk_prefix,
                       void* workspace, size_t workspace_bytes, artk_stream_t stream) {
  ARTK_CHECK_ARG(router_logits && topk_idx && topk_w && perm && inv_perm && row_token &&
                     expert_offsets && tile_prefix && blk_prefix,
                 "null pointer argument");
  ARTK_CHECK_ARG(T > 0 && E > 0 && k > 0 && k <= E, "T, E, k must be positive and k <= E");
  if (E > MOE_MAX_E || k > MOE_MAX_K || T * k >= (1ll << 30)) {
    set_error("supported: experts <= %d, top-k <= %d", MOE_MAX_E, MOE_MAX_K);
    return ARTK_ERR_UNSUPPORTED_SHAPE;
  }
  const int n = (int)(T * k);
  const int nb = (n + PERM_CHUNK - 1) / PERM_CHUNK;
  Workspace ws(workspace, workspace_bytes);
  int* cnt = ws.take<int>((size_t)nb * E);
  int* base = ws.take<int>((size_t)nb * E);
  if (!ws.ok()) {
    set_error("workspace too small: need %zu bytes, got %zu", ws.used, workspace_bytes);
    return ARTK_ERR_WORKSPACE_TOO_SMALL;
  }
  hipStream_t st = (hipStream_t)stream;
  moe_topk_kernel<<<(unsigned)((T + 3) / 4), 256, 0, st>>>(router_logits, T, E, k, topk_idx, topk_w);
  ARTK_CHECK_LAUNCH();
  moe_hist_kernel<<<nb, PERM_CHUNK, 0, st>>>(topk_idx, n, E, cnt);
  ARTK_CHECK_LAUNCH();
  moe_scan_kernel<<<1, SCAN_PARTS * MOE_MAX_E, 0, st>>>(cnt, nb, E, expert_offsets, base, tile_prefix, blk_prefix);
  ARTK_CHECK_LAUNCH();
  moe_scatter_kernel<<<nb, PERM_CHUNK, 0, st>>>(topk_idx, n, E, k, base, perm, inv_perm, row_token);
  ARTK_CHECK_LAUNCH();
  return ARTK_OK;
}

size_t artk_moe_lora_grouped_fwd_workspace_bytes(int64_t n_rows, int64_t in, int64_t out, int32_t E,
                                                 int32_t r) {
  (void)in;
  (void)out;
  (void)E;
  Workspace ws(nullptr, 0);
  ws.take<uint16_t>((size_t)n_rows * round16(r));
  return ws.used + 256;
}

int32_t artk_moe_lora_grouped_fwd(const void* x, const int32_t* gather, const void* W, const void* A,
                                  const void* B, float scale, const int32_t* expert_offsets,
                                  const int32_t* tile_prefix, const int32_t* blk_prefix,
                                  int64_t n_rows, int64_t in, int64_t out, int32_t E, int32_t r,
                                  void* y, float* xa, void* workspace, size_t workspace_bytes,
                                  artk_stream_t stream) {
  int32_t rc = check_moe(n_rows, in, out, E, r);
  if (rc) return rc;
  ARTK_CHECK_ARG(x && W && A && B && expert_offsets && tile_prefix && blk_prefix && y && xa,
                 "null pointer argument");
  ARTK_CHECK_ARG(aligned16(x) && aligned16(W) && aligned16(A) && aligned16(B) && aligned16(y),
                 "pointers must be 16-byte aligned");
  // gathered rows are addressed with 31-bit byte offsets from x; gather[i] < n_rows
  if (gather != nullptr && n_rows * in * 2 >= (1ll << 31)) {
    set_error("with a row gather, n_rows * in * 2 bytes (%lld) must stay below 2 GiB",
              (long long)(n_rows * in * 2));
    return ARTK_ERR_UNSUPPORTED_SHAPE;
  }
  const int RP = round16(r);
  Workspace ws(workspace, workspace_bytes);
  uint16_t* xa16 = ws.take<uint16_t>((size_t)n_rows * RP);
  if (!ws.ok()) {
    set_error("workspace too small: need %zu bytes, got %zu", ws.used, workspace_bytes);
    return ARTK_ERR_WORKSPACE_TOO_SMALL;
  }
  hipStream_t st = (hipStream_t)stream;
  if ((rc = launch_moe_rowdot(x, gather, (const uint16_t*)A, expert_offsets, blk_prefix, n_rows, E, in,
                              r, RP, scale, xa, xa16, st)))
    return rc;
  return launch_moe_gemm(W, x, gather, (const uint16_t*)B, xa16, y, expert_offsets, tile_prefix, n_rows,
                         out, in, E, r, RP, st);
}

// Scratch of the grouped backward, carved in the same order by the size query and the call.
struct MoeBwdScratch {
  uint16_t *Bt, *At, *gb16;
  float *gb, *rowp, *dummy;
};
static void carve_moe_bwd(Workspace& ws, int64_t n_rows, int64_t in, int64_t out, int E, int r, MoeBwdScratch& c) {
  const int RP = round16(r);
  c.Bt = ws.take<uint16_t>((size_t)E * r * out);  // [E,r,out]
  c.At = ws.take<uint16_t>((size_t)E * in * r);   // [E,in,r]
  c.gb = ws.take<float>((size_t)n_rows * r);
  c.gb16 = ws.take<uint16_t>((size_t)n_rows * RP);
  c.rowp = ws.take<float>((size_t)stats_grouped_chunks(out, r, E) * n_rows * r);
  c.dummy = ws.take<float>(1024);
}

size_t artk_moe_lora_grouped_bwd_workspace_bytes(int64_t n_rows, int64_t in, int64_t out, int32_t E,
                                                 int32_t r) {
  Workspace ws(nullptr, 0);
  MoeBwdScratch c;
  carve_moe_bwd(ws, n_rows, in, out, E, r, c);
  return ws.used + 256;
}

int32_t artk_moe_lora_grouped_bwd(const void* g, const void* x, const int32_t* gather, const void* W_t,
                                  const void* A, const void* B, const float* xa, float scale,
                                  const int32_t* expert_offsets, const int32_t* tile_prefix,
                                  const int32_t* blk_prefix, int64_t n_rows, int64_t in, int64_t out,
                                  int32_t E, int32_t r, void* dx, float* dA, float* dB,
                                  void* workspace, size_t workspace_bytes, artk_stream_t stream) {
  int32_t rc = check_moe(n_rows, in, out, E, r);
  if (rc) return rc;
  ARTK_CHECK_ARG(g && x && W_t && A && B && xa && expert_offsets && tile_prefix && blk_prefix && dx &&
                     dA && dB,
                 "null pointer argument");
  ARTK_CHECK_ARG(aligned16(g) && aligned16(x) && aligned16(W_t) && aligned16(A) && aligned16(B) && aligned16(dx) && aligned16(xa) &&
                     aligned16(dA) && aligned16(dB),
                 "pointers must be 16-byte aligned");
  if (n_rows * (in > out ? in : out) * 2 >= (1ll << 31)) {
    set_error("n_rows * max(in, out) * 2 bytes (%lld) must stay below 2 GiB (31-bit row offsets)",
              (long long)(n_rows * (in > out ? in : out) * 2));
    return ARTK_ERR_UNSUPPORTED_SHAPE;
  }
  const int RP = round16(r);
  Workspace ws(workspace, workspace_bytes);
  MoeBwdScratch c;
  carve_moe_bwd(ws, n_rows, in, out, E, r, c);
  if (!ws.ok()) {
    set_error("workspace too small: need %zu bytes, got %zu", ws.used, workspace_bytes);
    return ARTK_ERR_WORKSPACE_TOO_SMALL;
  }
  hipStream_t st = (hipStream_t)stream;
  if ((rc = launch_small_transpose2(B, c.Bt, E, out, r, A, c.At, E, r, in, st))) return rc;
  // one pass over g: g B_e per row (partials over column chunks) and dB_e = s g^T (x A_e^T) per expert
  if ((rc = launch_stats_grouped(g, n_rows, nullptr, n_rows, out, c.Bt, xa, r, E, expert_offsets, c.rowp, dB,
                                 scale, 0, c.dummy, st)))
    return rc;
  {
    StatsReduceJob ja{c.rowp, stats_grouped_chunks(out, r, E), n_rows, 1.f, c.gb, 0, c.gb16, RP, scale};
    StatsReduceJob jb{nullptr, 0, 0, 0.f, nullptr, 0, nullptr, 0, 0.f};
    if ((rc = launch_stats_reduce(ja, jb, r, st))) return rc;
  }
  if ((rc = launch_moe_gemm(W_t, g, nullptr, c.At, c.gb16, dx, expert_offsets, tile_prefix, n_rows, in, out,
                            E, r, RP, st)))
    return rc;
  // one pass over x (through the row gather when there is one): dA_e [r,in] = s (g B_e)^T x
  return launch_stats_grouped(x, gather ? (int64_t)0x3fffffff / in : n_rows, gather, n_rows, in, nullptr, c.gb, r,
                              E, expert_offsets, nullptr, dA, scale, 1, c.dummy, st);
}

int32_t artk_transpose_bf16_batched(const void* in, void* out, int64_t n, int64_t R, int64_t C,
                                    artk_stream_t stream) {
  ARTK_CHECK_ARG(in && out, "null pointer argument");
  ARTK_CHECK_ARG(n > 0 && n < 65536 && R > 0 && C > 0, "n, R, C must be positive (n < 65536)");
  dim3 grid((unsigned)((C + 63) / 64), (unsigned)((R + 63) / 64), (unsigned)n);
  transpose_bf16_batched_kernel<<<grid, 256, 0, (hipStream_t)stream>>>((const uint16_t*)in,
                                                                       (uint16_t*)out, R, C);
  ARTK_CHECK_LAUNCH();
  return ARTK_OK;
}

}  // extern "C"
