// GRPO logprob / loss hot path for gfx950: lm_head projection with online
// log-sum-exp and target gather, clipped-surrogate loss with its gradient
// coefficient, softmax gradient and the d_hidden GEMM.
//
// Reference behaviour that these kernels restate:
//   src/art/local/train.py:245-281  chunked matmul -> gather -> logsumexp
//   src/art/local/train.py:284-285  shift_tensor (folded into index math here)
//   src/art/local/train.py:111-151  ratio / clip / KL / weight*mask / normalise
#include "common.hpp"
#include "gemm_nt.hpp"
#include "gemm_plain8.hpp"

#include <math.h>

#include <mutex>

namespace artk {

// Work-group shape of each GEMM kernel (see gemm_nt.hpp).
constexpr int FWD_NI = 2;   // lm_head projection + log-sum-exp epilogue: 8 waves
constexpr int BWD_NI = 2;   // d_hidden GEMM
constexpr int GEMM_NI = 2;  // plain GEMM: 8 waves, the first wave of each SIMD issues the DMA (gemm_plain8.hpp)

// ----------------------------------------------------------------------------
// index helpers
// ----------------------------------------------------------------------------

// Element of a per-token input seen by position t: with shift, element t+1 of
// the same row of the [B,S] input, or the pad value at the row's last position.
__device__ __forceinline__ bool shifted_index(int64_t t, int64_t S, int shift, int64_t& src) {
  if (!shift) {
    src = t;
    return true;
  }
  int64_t s = t % S;
  src = t + 1;
  return s + 1 < S;
}

__device__ __forceinline__ int64_t target_id(const int64_t* ids, int64_t t, int64_t S, int shift) {
  int64_t src;
  return shifted_index(t, S, shift, src) ? ids[src] : (int64_t)0;  // pad id 0 (train.py:79)
}

// The rows of one chunk.  Dense mode: row r is position t0 + r and there are
// `cap` of them.  Compact mode (the forward is evaluated only for positions that
// can contribute to the loss): row r is position row_token[r] and the number of
// rows is min(cap, *n_all - c0), known only on the device; kernels are launched
// for `cap` rows and the surplus work-groups / threads exit at once.
struct ChunkRows {
  const int* row_token;  // nullptr in dense mode; else already offset to the chunk's first row
  const int* n_all;      // compact mode: number of compact rows of the whole batch
  int64_t t0;
  int c0, cap;
  __device__ __forceinline__ int n() const {
    if (n_all == nullptr) return cap;
    int left = *n_all - c0;
    return left < 0 ? 0 : (left < cap ? left : cap);
  }
  __device__ __forceinline__ int64_t token(int r) const {
    return row_token ? (int64_t)row_token[r] : t0 + r;
  }
};

// ----------------------------------------------------------------------------
// K1: logits tile = lm_head[256 vocab rows] x hidden[256 positions]^T, with
// per-position (max, sum-exp) partials over the tile's vocab rows, gather of
// the target logit, and (optionally) the bf16 logits stored to a scratch.
// ----------------------------------------------------------------------------
struct FwdParams {
  const void* hidden;   // bf16 [*,H]: dense: first row = position t0; compact: position 0
  const void* W;        // [V,H] bf16
  const int64_t* ids;   // [T] (whole batch)
  ChunkRows rows;
  int64_t Tc;           // row pitch of part / sel (= rows.cap)
  int64_t S, V, H;
  int shift;
  float2* part;         // [2*VT][Tc]  (max, sumexp)
  float* sel;           // [Tc]        selected logit (pre-filled with NaN)
  uint16_t* stash;      // [Tc,V] bf16 or nullptr: exp(logit - ref[row]) of the rows the backward reads
  const float* ref;     // [Tc] reference logit of each row (stash only): the target's own logit
  const uint8_t* need;  // [Tc] rows of the stash that the backward will read; nullptr: all
  int VT, TT;
};

// Epilogue of one logits tile, per wave: its 128 vocabulary rows x 64 positions.
//
// For every position: the (reference, sum-exp) partial over the wave's vocabulary rows and the
// gather of the target logit.  The reference of the partial is the maximum of the 128 logits,
// except for a position whose row goes to the stash: there it is the row's own reference
// ref[row], so that one exponential per logit, exp(z - ref), serves both the sum and the
// stash (the exponentials are the epilogue's cost: they run at a quarter of the vector rate
// while the matrix pipe idles).  Partials of one position merge whatever their references are.
// If a logit exceeds its row's reference by more than fp32's exponent range the sum is
// infinite; such a position's partial is recomputed against the maximum (its stash row holds
// infinities and the backward drops the row, see splitk_reduce_kernel).
//
// STASH: bf16 exp(z - ref) of the positions in `need`.  A lane holds 4 consecutive vocabulary
// rows of one position, so stored straight from the registers a row would go out in 8-byte
// pieces, 32 positions per store instruction: the L2 then takes one 16-byte request per piece
// pair and the wave waits for thousands of them.  Instead the wave transposes 32 positions at
// a time through `scratch` (EPI_LDS_PER_WAVE bytes of LDS per wave that nothing else uses during
// the epilogue: 32 rows of 256 bytes at a pitch of 272, which keeps the 8-byte writes and the
// 16-byte reads free of bank conflicts), and 16 lanes store 256 contiguous bytes of a position.
// RAGGED: the tile reaches past the last vocabulary row and those rows are left out.
struct EpiRow {  // what the epilogue needs to know about one position of the tile
  int64_t y;     // target id, -1 past the end
  int col;
  bool want;
  float ref;
};
// Issued before the next tile's first DMA stage, so that waiting for these values does not wait
// for that stage (loads complete in order).
template <bool STASH>
__device__ __forceinline__ void lmhead_epilogue_rows(const FwdParams& p, int tt, int n, EpiRow (&row)[FWD_NI]) {
  const int lane = threadIdx.x & 63;
  const int wn = wave_n<FWD_NI>(threadIdx.x >> 6);
#pragma unroll
  for (int ni = 0; ni < FWD_NI; ++ni) {
    EpiRow& r = row[ni];
    r.col = tt * TILE + acc_col<FWD_NI>(wn, ni, lane);
    r.y = r.col < n ? target_id(p.ids, p.rows.token(r.col), p.S, p.shift) : (int64_t)-1;
    r.want = STASH && r.col < n && (p.need == nullptr || p.need[r.col] != 0);
    r.ref = r.want ? p.ref[r.col] : 0.f;
  }
}

template <bool STASH, bool RAGGED>
__device__ __forceinline__ void lmhead_fwd_epilogue_impl(const TileAcc<FWD_NI>& acc, const FwdParams& p, int vt,
                                                         int tt, int n, const EpiRow (&row)[FWD_NI],
                                                         char* scratch) {
  static_assert(FWD_NI == 2, "the LDS transpose is laid out for 8 waves of 128 x 64");
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int wm = wave_m<FWD_NI>(wave), wn = wave_n<FWD_NI>(wave);
  const int half = lane >> 5;
  const int c = lane & 31;
  const int64_t vbase = (int64_t)vt * TILE + wm * 128;  // first vocab row of this wave
  const int vleft = (int)(p.V - vbase < 128 ? p.V - vbase : 128);  // valid rows of this wave (may be <= 0)
  char* my = scratch + wave * EPI_LDS_PER_WAVE;
  char* my_w = my + c * EPI_PITCH + half * 8;                              // this lane's 8-byte pieces
  const char* my_r = my + (lane >> 4) * EPI_PITCH + (lane & 15) * 16;      // 16 bytes of row i*4 + lane/16

#pragma unroll
  for (int ni = 0; ni < FWD_NI; ++ni) {
    // A position's 128 logits of this wave: 64 in this lane, 64 in lane^32.
    float m = -INFINITY;
#pragma unroll
    for (int mi = 0; mi < 4; ++mi)
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        const int r = mi * 32 + (j >> 2) * 8 + half * 4 + (j & 3);
        const float z = acc.c[mi][ni][j];
        m = fmaxf(m, (RAGGED && r >= vleft) ? -INFINITY : z);
      }
    m = fmaxf(m, __shfl_xor(m, 32, 64));
    float mr = row[ni].want ? row[ni].ref : m;  // reference of this position's partial
    const float mb = (mr == -INFINITY ? 0.f : mr) * LOG2E;
    float l = 0.f;
#pragma unroll
    for (int mi = 0; mi < 4; ++mi)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        float e[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const int r = mi * 32 + q * 8 + half * 4 + k;
          e[k] = __builtin_amdgcn_exp2f(__builtin_fmaf(acc.c[mi][ni][q * 4 + k], LOG2E, -mb));
          if (RAGGED && r >= vleft) e[k] = 0.f;
          l += e[k];
        }
        if (STASH) {
          bf16x4 o;
#pragma unroll
          for (int k = 0; k < 4; ++k) o[k] = (__bf16)e[k];
          *(bf16x4*)(my_w + (mi * 8 + q * 2) * 8) = o;  // rows mi*32 + q*8 + half*4 .. +3 of position c
        }
      }
    l += __shfl_xor(l, 32, 64);
    if (STASH) {
      const bool ovf = row[ni].want && !(l <= 3.0e38f);
      if (__any(ovf)) {
        const float mb2 = (m == -INFINITY ? 0.f : m) * LOG2E;
        float l2 = 0.f;
#pragma unroll
        for (int mi = 0; mi < 4; ++mi)
#pragma unroll
          for (int j = 0; j < 16; ++j) {
            const int r = mi * 32 + (j >> 2) * 8 + half * 4 + (j & 3);
            const float e = __builtin_amdgcn_exp2f(__builtin_fmaf(acc.c[mi][ni][j], LOG2E, -mb2));
            l2 += (RAGGED && r >= vleft) ? 0.f : e;
          }
        l2 += __shfl_xor(l2, 32, 64);
        if (ovf) {
          mr = m;
          l = l2;
        }
      }
    }
    if (lane < 32 && row[ni].col < n)
      p.part[(int64_t)(vt * 2 + wm) * p.Tc + row[ni].col] = make_float2(mr, l);

    // Gather: exactly one lane of one wave of the whole grid holds logit[y].
    const int64_t rel = row[ni].y - vbase;
    const bool hit = rel >= 0 && rel < 128 && ((((int)rel) >> 2) & 1) == half;
    if (__any(hit)) {
      float s = 0.f;
#pragma unroll
      for (int mi = 0; mi < 4; ++mi)
#pragma unroll
        for (int j = 0; j < 16; ++j) {
          const int r = mi * 32 + (j >> 2) * 8 + half * 4 + (j & 3);
          s = (r == (int)rel) ? acc.c[mi][ni][j] : s;
        }
      if (hit) p.sel[row[ni].col] = s;
    }

    if (STASH) {
      const uint32_t mask = (uint32_t)__ballot(row[ni].want);  // bit i: position i of these 32 (both halves agree)
      if (mask != 0) {
        __builtin_amdgcn_wave_barrier();
        const int k16 = lane & 15;
        const int64_t v0 = vbase + k16 * 8;
        const int64_t col0 = (int64_t)tt * TILE + wn * 64 + ni * 32;
        uint16_t* dst = p.stash + (col0 + (lane >> 4)) * p.V + v0;
        const uint32_t mine = v0 < p.V ? mask >> (lane >> 4) : 0u;  // bit 4i: position i*4 + lane/16
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          uint4 d[4];
#pragma unroll
          for (int i = 0; i < 4; ++i) d[i] = *(const uint4*)(my_r + (h * 4 + i) * 4 * EPI_PITCH);
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if ((mine >> (4 * (h * 4 + i))) & 1u) *(uint4*)(dst + (int64_t)(h * 4 + i) * 4 * p.V) = d[i];
        }
        __builtin_amdgcn_wave_barrier();
      }
    }
  }
}

template <bool STASH>
__device__ __forceinline__ void lmhead_fwd_epilogue(const TileAcc<FWD_NI>& acc, const FwdParams& p, int vt,
                                                    int tt, int n, const EpiRow (&row)[FWD_NI], char* scratch) {
  // The accumulators are only read (writing to them would make the compiler shuttle all of
  // them between the accumulation and the vector registers).
  if ((int64_t)vt * TILE + TILE > p.V)
    lmhead_fwd_epilogue_impl<STASH, true>(acc, p, vt, tt, n, row, scratch);
  else
    lmhead_fwd_epilogue_impl<STASH, false>(acc, p, vt, tt, n, row, scratch);
}

// The order of the tiles of one launch: TT position tiles that hold rows (in compact mode their
// number is known only on the device) and how many vocabulary tiles an XCD's 32 work-groups walk
// per position tile.  With plenty of position tiles a patch is 4 x 8 (gemm_nt.hpp); with fewer
// than a patch is wide it takes more vocabulary tiles instead, so that the 32 still work on one
// patch (measured at 2048 x 896 x 151936: 8 position tiles 0.897 -> 0.876 ms per step with 8
// instead of 4, the 4 position tiles of its compact rows 0.861 -> 0.644 ms; at 3584 and 21-22
// position tiles 4 stays best, 20.4 against 20.8 ms).
struct FwdOrder {
  int TT, n_tiles, group;
  __device__ __forceinline__ FwdOrder(const FwdParams& p, int n) {
    const int live = (n + TILE - 1) / TILE;
    TT = live < p.TT ? live : p.TT;
    n_tiles = p.VT * TT;
    group = TT >= 12 ? TILE_GROUP_STREAMING : (TT >= 4 ? 8 : (TT >= 2 ? 16 : 32));
  }
  // Tile id t (< n_tiles) -> vocabulary tile, position tile.
  __device__ __forceinline__ void coords(const FwdParams& p, int t, int& vt, int& tt) const {
    tile_coords(xcd_remap(t, n_tiles), p.VT, TT, vt, tt, group);
  }
};

// Persistent work-groups (one per CU): each walks tiles t, t + grid, ...  The
// next tile's loaders are set up before the current tile's main loop and its
// first DMA stage is started before the current tile's epilogue, so the
// prologue latency of a tile hides behind the epilogue of the previous one.
// Loaders and main loop of one forward tile.  GATHER: the rows of the chunk are compact (row_token
// maps them to positions and the hidden states are gathered); otherwise both operands are plain
// panels and the first wave of each SIMD issues all DMA (gemm_plain8.hpp).
template <bool GATHER>
struct FwdLoaders : PlainTileLoaders {
  __device__ __forceinline__ void init_tile(const FwdParams& p, int vt, int tt, int n) {
    init(p.W, p.H, (int64_t)vt * TILE, p.V, p.hidden, p.H, (int64_t)tt * TILE, n, 0, (int)p.H);
  }
  __device__ __forceinline__ void run(TileAcc<FWD_NI>& acc, char* smem) const {
    gemm_tile_run_plain8<false>(acc, smem, *this);
  }
};
template <>
struct FwdLoaders<true> : TileLoaders<FWD_NI> {
  __device__ __forceinline__ void init_tile(const FwdParams& p, int vt, int tt, int n) {
    init(p.W, p.H, (int64_t)vt * TILE, p.V, p.hidden, p.H, (int64_t)tt * TILE, n, 0, (int)p.H, p.rows.row_token);
  }
  __device__ __forceinline__ void run(TileAcc<FWD_NI>& acc, char* smem) const {
    gemm_tile_run<FWD_NI, FWD_NI, false>(acc, smem, static_cast<const TileLoaders<FWD_NI>&>(*this));
  }
};

template <bool STASH, bool GATHER>
__global__ __launch_bounds__(nthreads<FWD_NI>()) void lmhead_fwd_kernel(FwdParams p) {
  __shared__ __attribute__((aligned(1024))) char smem[GEMM_LDS_BYTES + (STASH ? EPI_LDS_EXTRA : 0)];
  const int n = p.rows.n();
  const FwdOrder order(p, n);
  int t = blockIdx.x, vt, tt;
  if (t >= order.n_tiles) return;
  order.coords(p, t, vt, tt);
  {
    FwdLoaders<GATHER> first;
    first.init_tile(p, vt, tt, n);
    first.issue_first(smem);
  }
  for (;;) {
    const int t2 = t + gridDim.x;
    int vt2 = 0, tt2 = 0;
    const bool more = t2 < order.n_tiles;
    if (more) order.coords(p, t2, vt2, tt2);
    TileAcc<FWD_NI> acc;
    acc.zero();
    {
      FwdLoaders<GATHER> cur;  // its first stage is already on the way
      cur.init_tile(p, vt, tt, n);
      cur.run(acc, smem);
    }
    EpiRow row[FWD_NI];
    lmhead_epilogue_rows<STASH>(p, tt, n, row);
    if (more) {
      // loaders are rebuilt rather than kept: alive through the epilogue they cost registers
      FwdLoaders<GATHER> nxt;
      nxt.init_tile(p, vt2, tt2, n);
      nxt.issue_first(smem);
    }
    // the second LDS stage (and what lies behind it) is idle until the next tile's first barrier:
    // scratch of the epilogue
    lmhead_fwd_epilogue<STASH>(acc, p, vt, tt, n, row, smem + STAGE_BYTES);
    if (!more) break;
    t = t2;
    vt = vt2;
    tt = tt2;
  }
}

// K2: merge the per-tile (max, sumexp) partials of each position.  A block
// handles 16 positions; 16 threads per position each merge a strided share of
// the partials online, then the 16 shares are merged through LDS.
// logprob is indexed by position (whole batch), lse by chunk row.
__global__ __launch_bounds__(256) void lse_finalize_kernel(const float2* __restrict__ part,
                                                           int nparts, int64_t Tc, ChunkRows rows,
                                                           const float* __restrict__ sel,
                                                           float* __restrict__ logprob,
                                                           float* __restrict__ lse) {
  __shared__ float2 red[16][17];
  const int tl = threadIdx.x & 15, sl = threadIdx.x >> 4;
  const int64_t t = (int64_t)blockIdx.x * 16 + tl;
  const int n = rows.n();
  float m = -INFINITY, l = 0.f;
  if (t < n) {
    // eight loads in flight per thread (the merge itself is a dependent chain), same merge order
    for (int i0 = sl; i0 < nparts; i0 += 16 * 8) {
      float2 v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int i = i0 + 16 * u;
        v[u] = i < nparts ? part[(int64_t)i * Tc + t] : make_float2(-INFINITY, 0.f);
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        if (i0 + 16 * u >= nparts) break;
        const float mn = fmaxf(m, v[u].x);
        if (mn != -INFINITY)
          l = l * __builtin_amdgcn_exp2f((m - mn) * LOG2E) + v[u].y * __builtin_amdgcn_exp2f((v[u].x - mn) * LOG2E);
        m = mn;
      }
    }
  }
  red[sl][tl] = make_float2(m, l);
  __syncthreads();
  if (sl == 0 && t < n) {
    float M = -INFINITY;
#pragma unroll
    for (int i = 0; i < 16; ++i) M = fmaxf(M, red[i][tl].x);
    float L = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const float2 v = red[i][tl];
      if (v.x != -INFINITY) L += v.y * __builtin_amdgcn_exp2f((v.x - M) * LOG2E);
    }
    const float z = M + logf(L);
    lse[t] = z;
    if (logprob) logprob[rows.token((int)t)] = sel[t] - z;
  }
}

// need[i] = 1 when position t0+i can have a non-zero loss coefficient: its
// (shifted) mask is set and weight and advantage are non-zero.
__global__ __launch_bounds__(256) void need_from_inputs_kernel(const uint8_t* __restrict__ mask,
                                                               const float* __restrict__ weights,
                                                               const float* __restrict__ adv,
                                                               const float* __restrict__ ref_lp,
                                                               int64_t t0, int64_t n, int64_t S,
                                                               int shift, uint8_t* __restrict__ need) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  int64_t src;
  uint8_t v = 0;
  if (shifted_index(t0 + i, S, shift, src))
    v = mask[src] != 0 && weights[src] != 0.f && (adv[src] != 0.f || ref_lp != nullptr);
  need[i] = v;
}

__global__ __launch_bounds__(256) void need_from_grad_kernel(const float* __restrict__ g, int64_t n,
                                                             uint8_t* __restrict__ need) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) need[i] = g[i] != 0.f;
}

// Positions of the whole batch that can have a non-zero loss coefficient (same
// test as need_from_inputs_kernel), ascending, and their number.  One block.
__global__ __launch_bounds__(1024) void compact_eval_kernel(const uint8_t* __restrict__ mask,
                                                            const float* __restrict__ weights,
                                                            const float* __restrict__ adv,
                                                            const float* __restrict__ ref_lp, int64_t T,
                                                            int64_t S, int shift,
                                                            int* __restrict__ eval_idx,
                                                            int* __restrict__ n_eval) {
  __shared__ int wave_tot[16];
  const int64_t per = (T + 1023) / 1024;
  const int64_t r0 = threadIdx.x * per;
  auto wanted = [&](int64_t t) {
    int64_t src;
    return shifted_index(t, S, shift, src) && mask[src] != 0 && weights[src] != 0.f &&
           (adv[src] != 0.f || ref_lp != nullptr);
  };
  int cnt = 0;
  for (int64_t i = 0; i < per; ++i)
    if (r0 + i < T && wanted(r0 + i)) ++cnt;
  int incl = cnt;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    int v = __shfl_up(incl, o, 64);
    if ((threadIdx.x & 63) >= o) incl += v;
  }
  if ((threadIdx.x & 63) == 63) wave_tot[threadIdx.x >> 6] = incl;
  __syncthreads();
  if (threadIdx.x == 0) {
    int run = 0;
    for (int w = 0; w < 16; ++w) {
      int v = wave_tot[w];
      wave_tot[w] = run;
      run += v;
    }
    *n_eval = run;
  }
  __syncthreads();
  int at = wave_tot[threadIdx.x >> 6] + incl - cnt;
  for (int64_t i = 0; i < per; ++i)
    if (r0 + i < T && wanted(r0 + i)) eval_idx[at++] = (int)(r0 + i);
}

__global__ void fill_f32_kernel(float* p, int64_t n, float v) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = v;
}

// ----------------------------------------------------------------------------
// Loss kernels
// ----------------------------------------------------------------------------

// count[0] = number of positions whose (shifted) assistant mask is set; count[1] = 0. One block.
__global__ __launch_bounds__(1024) void mask_count_kernel(const uint8_t* __restrict__ mask,
                                                          int64_t T, int64_t S, int shift,
                                                          int* __restrict__ count) {
  __shared__ int red[16];
  int c = 0;
  for (int64_t t = threadIdx.x; t < T; t += 1024) {
    int64_t src;
    if (shifted_index(t, S, shift, src)) c += mask[src] != 0;
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) c += __shfl_xor(c, o, 64);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = c;
  __syncthreads();
  if (threadIdx.x == 0) {
    int s = 0;
    for (int i = 0; i < 16; ++i) s += red[i];
    count[0] = s;
    count[1] = 0;  // rows dropped by splitk_reduce_kernel (fused step only)
  }
}

struct LossParams {
  const float* new_lp;   // [T] by position (whole batch)
  const float* old_lp;   // [T] whole batch (frame given by shift)
  const float* adv;      // [T]
  const uint8_t* mask;   // [T]
  const float* weights;  // [T]
  const float* ref_lp;   // [T] by position, or nullptr
  const int* count;      // mask count of the whole batch
  ChunkRows rows;
  int64_t S;
  int shift;
  float clip_lo, clip_hi, beta;
  float* pl_tok;         // [T] by position: weighted policy-loss term
  float* kl_tok;         // [T] by position: weighted KL term
  float* coef;           // [rows.cap] by chunk row: d loss / d new_lp, or nullptr
};

__global__ __launch_bounds__(256) void grpo_loss_tok_kernel(LossParams p) {
  int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= p.rows.n()) return;
  const int64_t t = p.rows.token((int)i);
  int64_t src;
  const bool in = shifted_index(t, p.S, p.shift, src);
  float oldv = in ? p.old_lp[src] : 0.f;
  const float adv = in ? p.adv[src] : 0.f;
  const float w = in ? p.weights[src] : 0.f;
  const float m = (in && p.mask[src] != 0) ? 1.f : 0.f;
  const float nw = p.new_lp[t];
  if (isnan(oldv)) oldv = nw;  // missing old logprob: sampled under the current policy
  const float ratio = expf(nw - oldv);
  const float a = ratio * adv;
  const float clipped = fminf(fmaxf(ratio, p.clip_lo), p.clip_hi);
  const float b = clipped * adv;
  const float pl = -fminf(a, b);
  // Gradient of -min(a, b) w.r.t. new_lp. Inside the clip range a and b are the
  // same number and both pass the gradient; outside only a does, when it is the min.
  const bool inside = ratio >= p.clip_lo && ratio <= p.clip_hi;
  float g = (inside || a < b) ? -a : 0.f;
  float kl = 0.f;
  if (p.ref_lp != nullptr) {
    const float d = p.ref_lp[t] - nw;
    const float e = expf(d);
    kl = e - d - 1.f;
    g += p.beta * (1.f - e);
  }
  const float denom = (float)(*p.count) + 1e-6f;
  const float wm = w * m;
  p.pl_tok[t] = pl * wm;
  p.kl_tok[t] = kl * wm;
  if (p.coef) p.coef[i] = (wm != 0.f) ? g * wm / denom : 0.f;
}

// scalars = {loss, mean_policy_loss, mean_kl, mask_count} and, with `with_dropped` (the fused
// step), scalars[4] = count[1], the rows whose gradient was dropped.  One block; fixed
// summation order, so the result is bit-reproducible run to run.
__global__ __launch_bounds__(1024) void grpo_loss_reduce_kernel(const float* __restrict__ pl_tok,
                                                                const float* __restrict__ kl_tok,
                                                                int64_t T,
                                                                const int* __restrict__ count,
                                                                float beta, int with_dropped,
                                                                float* __restrict__ scalars) {
  __shared__ double red[2][16];
  double a = 0.0, b = 0.0;
  for (int64_t t = threadIdx.x; t < T; t += 1024) {
    a += (double)pl_tok[t];
    b += (double)kl_tok[t];
  }
  a = wave_sum(a);
  b = wave_sum(b);
  if ((threadIdx.x & 63) == 0) {
    red[0][threadIdx.x >> 6] = a;
    red[1][threadIdx.x >> 6] = b;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    double sa = 0.0, sb = 0.0;
    for (int i = 0; i < 16; ++i) {
      sa += red[0][i];
      sb += red[1][i];
    }
    const float denom = (float)(*count) + 1e-6f;
    const float mpl = (float)sa / denom;
    const float mkl = (float)sb / denom;
    scalars[0] = mpl + beta * mkl;
    scalars[1] = mpl;
    scalars[2] = mkl;
    scalars[3] = (float)(*count);
    if (with_dropped) scalars[4] = (float)count[1];
  }
}

// ----------------------------------------------------------------------------
// K3a: active rows of a chunk (coef != 0) in ascending order, the inverse map,
// and the schedule of the d_hidden GEMM over those rows.  One block.
//   sched[0] = n_active, [1] = token tiles, [2] = K splits, [3] = work-groups
// Rows whose coefficient is zero (non-assistant positions, zero advantage) have
// an exactly zero d_hidden row and are skipped by K4.
__global__ __launch_bounds__(1024) void compact_rows_kernel(const float* __restrict__ coef,
                                                            ChunkRows rows, int HT, int ksteps,
                                                            int part_rows,
                                                            int num_cus, int* __restrict__ active_idx,
                                                            int* __restrict__ pos,
                                                            int* __restrict__ sched) {
  __shared__ int wave_tot[16];
  __shared__ int total;
  const int Tc = rows.n();
  const int per = (rows.cap + 1023) / 1024;
  const int r0 = threadIdx.x * per;
  int cnt = 0;
  for (int i = 0; i < per; ++i) {
    int r = r0 + i;
    if (r < Tc && coef[r] != 0.f) ++cnt;
  }
  // exclusive scan of cnt over the block
  int incl = cnt;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    int v = __shfl_up(incl, o, 64);
    if ((threadIdx.x & 63) >= o) incl += v;
  }
  if ((threadIdx.x & 63) == 63) wave_tot[threadIdx.x >> 6] = incl;
  __syncthreads();
  if (threadIdx.x == 0) {
    int run = 0;
    for (int w = 0; w < 16; ++w) {
      int v = wave_tot[w];
      wave_tot[w] = run;
      run += v;
    }
    total = run;
  }
  __syncthreads();
  int at = wave_tot[threadIdx.x >> 6] + incl - cnt;
  for (int i = 0; i < per; ++i) {
    int r = r0 + i;
    if (r >= Tc) break;
    if (coef[r] != 0.f) {
      active_idx[at] = r;
      pos[r] = at;
      ++at;
    } else {
      pos[r] = -1;
    }
  }
  if (threadIdx.x == 0) {
    const int n = total;
    const int tta = (n + TILE - 1) / TILE;
    const int tiles = HT * tta;
    int best = 1;
    float best_eff = 0.f;
    for (int ns = 1; ns <= 16 && tiles > 0; ++ns) {
      if (ns > 1 && (ksteps / ns < 32 || ns * tta * TILE > part_rows)) break;
      int blocks = tiles * ns;
      int rounds = (blocks + num_cus - 1) / num_cus;
      float eff = (float)blocks / ((float)rounds * num_cus);
      if (eff > best_eff + 0.02f) {
        best_eff = eff;
        best = ns;
      }
    }
    sched[0] = n;
    sched[1] = tta;
    sched[2] = best;
    sched[3] = tiles * best;
  }
}

// K0 (before the forward of a chunk the backward will read): ref[r] = logit of row r's own
// target, hidden[token(r)] . lm_head[y_r], in fp32; 0 for rows the backward does not need or
// whose target is not a vocabulary id.  The forward stashes exp(logit - ref[r]) instead of the
// logit: softmax is invariant to the shift, the target was sampled from (nearly) this
// distribution, so its logit is a reference within a few tens of nats of the row's maximum,
// and bf16 has the exponent range of fp32 — exp(z - ref) is representable unless a logit
// exceeds the target's by 88 nats; a row whose lse exceeds its reference by more than 80 nats
// (a sampled token of probability below e^-80 under the current policy) is dropped by
// splitk_reduce_kernel: zero gradient, counted.  With the exponentials in the stash the softmax gradient needs no
// pass of its own: d_hidden[t] = coef_t (W[y_t] - exp(ref_t - lse_t) sum_v e[t,v] W[v]),
// the sum being the GEMM K4 and the rest the epilogue of K5.  (A stash of logits needed a
// 2 x [Tc_active, V] read-modify-write between K2 and K4 to turn them into gradients.)
// One wave per row.
__global__ __launch_bounds__(256) void target_ref_kernel(const uint16_t* __restrict__ hidden,
                                                         const uint16_t* __restrict__ W,
                                                         const int64_t* __restrict__ ids, ChunkRows rows,
                                                         const uint8_t* __restrict__ need, int64_t S,
                                                         int shift, int64_t V, int64_t H,
                                                         float* __restrict__ ref) {
  const int lane = threadIdx.x & 63;
  const int r = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (r >= rows.n()) return;
  float s = 0.f;
  const int64_t y = target_id(ids, rows.token(r), S, shift);
  if ((need == nullptr || need[r] != 0) && y >= 0 && y < V) {
    // `hidden` starts at the chunk's first row when the rows are dense, at position 0 when they
    // are gathered
    const uint16_t* h = hidden + (int64_t)(rows.row_token ? rows.token(r) : r) * H;
    const uint16_t* w = W + y * H;
    for (int64_t k = lane * 8; k < H; k += 512) {
      const uint4 a = *(const uint4*)(h + k), b = *(const uint4*)(w + k);
      const uint32_t av[4] = {a.x, a.y, a.z, a.w}, bv[4] = {b.x, b.y, b.z, b.w};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        s = __builtin_fmaf(__uint_as_float(av[e] << 16), __uint_as_float(bv[e] << 16), s);
        s = __builtin_fmaf(__uint_as_float(av[e] & 0xffff0000u), __uint_as_float(bv[e] & 0xffff0000u), s);
      }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o, 64);
  }
  if (lane == 0) ref[r] = s;
}

// ----------------------------------------------------------------------------
// K4: d_hidden tile = P[256 positions, k-range of V] x lm_head_t[256 h, same]^T
// ----------------------------------------------------------------------------
struct BwdParams {
  const void* Wt;          // [H,V] bf16
  const void* P;           // [Tc,V] bf16 (only active rows hold gradients)
  int64_t V, H;
  int HT;
  const int* active_idx;   // [n_active] rows of P, ascending
  const int* sched;        // see compact_rows_kernel
  float* partial;          // [nsplit][tiles*256][H] f32
};

// The grid is sized for the worst case (every row active); the work-groups
// beyond the device-side schedule exit at once.
__global__ __launch_bounds__(nthreads<BWD_NI>()) void dhidden_gemm_kernel(BwdParams p) {
  __shared__ __attribute__((aligned(1024))) char smem[GEMM_LDS_BYTES];
  const int n_active = p.sched[0], TT = p.sched[1], nsplit = p.sched[2], n_work = p.sched[3];
  if ((int)blockIdx.x >= n_work) return;
  const int id = xcd_remap(blockIdx.x, n_work);
  const int tiles = p.HT * TT;
  const int split = id / tiles;
  const int rem = id - split * tiles;
  int ht, tt;
  tile_coords(rem, p.HT, TT, ht, tt);
  const int KT = (int)(p.V / BK);
  const int kb = (int)((int64_t)split * KT / nsplit);
  const int ke = (int)((int64_t)(split + 1) * KT / nsplit);

  TileAcc<BWD_NI> acc;
  acc.zero();
  gemm_tile_nt(acc, smem, p.Wt, p.V, (int64_t)ht * TILE, p.H, p.P, p.V, (int64_t)tt * TILE,
               n_active, kb * BK, ke * BK, p.active_idx);

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int wm = wave_m<BWD_NI>(wave), wn = wave_n<BWD_NI>(wave);
  const int half = lane >> 5;
  const int64_t rows_per_split = (int64_t)TT * TILE;
#pragma unroll
  for (int ni = 0; ni < BWD_NI; ++ni) {
    const int col = tt * TILE + acc_col<BWD_NI>(wn, ni, lane);  // compact row
    if (col >= n_active) continue;
#pragma unroll
    for (int mi = 0; mi < 4; ++mi)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int64_t h = (int64_t)ht * TILE + wm * 128 + mi * 32 + q * 8 + half * 4;
        if (h >= p.H) continue;
        floatx4 o;
#pragma unroll
        for (int e = 0; e < 4; ++e) o[e] = acc.c[mi][ni][q * 4 + e];
        *(floatx4*)(p.partial + ((int64_t)split * rows_per_split + col) * p.H + h) = o;
      }
  }
}

constexpr float STASH_MAX_NATS = 80.f;

// K5: d_hidden row of chunk row r: 0 for inactive rows, else
//   bf16( coef_r * ( W[y_r] - exp(ref_r - lse_r) * G ) ),  G = sum over splits of partial[active slot of r]
// (G = sum_v exp(z[r,v] - ref_r) W[v], see target_ref_kernel); 4 elements per thread.  `out` is
// the whole batch's d_hidden, indexed by position.
// A row with lse_r - ref_r above STASH_MAX_NATS (its target has probability below e^-80 under
// the current policy) is dropped: sum_v exp(z - ref) = exp(lse - ref) bounds every stashed
// exponential and, times max |W|, every element of G, so up to the limit all of them are finite
// in bf16 / fp32, and beyond it they may be inf or NaN.  Such a row gets a zero gradient (what
// the reference would compute for it is cf * (W[y] - p W) with p ~ one-hot elsewhere: a finite
// row; dropping it keeps the step finite) and is counted in *dropped (may be null).
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ partial,
                                                            const int* __restrict__ pos,
                                                            const int* __restrict__ sched,
                                                            ChunkRows rows, int64_t H, int64_t V,
                                                            const float* __restrict__ coef,
                                                            const float* __restrict__ lse,
                                                            const float* __restrict__ ref,
                                                            const int64_t* __restrict__ ids, int64_t S,
                                                            int shift, const uint16_t* __restrict__ W,
                                                            uint16_t* __restrict__ out,
                                                            int* __restrict__ dropped) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t h4 = H / 4;
  if (i >= (int64_t)rows.n() * h4) return;
  const int64_t r = i / h4, c = i - r * h4;
  const int pr = pos[r];
  floatx4 s = {0.f, 0.f, 0.f, 0.f};
  const bool over = pr >= 0 && !(lse[r] - ref[r] <= STASH_MAX_NATS);  // also true for NaN
  if (over) {
    if (c == 0 && dropped != nullptr) atomicAdd(dropped, 1);
  } else if (pr >= 0) {
    const int nsplit = sched[2];
    const int64_t rows_per_split = (int64_t)sched[1] * TILE;
    for (int k = 0; k < nsplit; ++k)
      s += ((const floatx4*)(partial + ((int64_t)k * rows_per_split + pr) * H))[c];
    const float cf = coef[r];
    const float scale = __builtin_amdgcn_exp2f((ref[r] - lse[r]) * LOG2E);
    const int64_t y = target_id(ids, rows.token((int)r), S, shift);
    floatx4 w = {0.f, 0.f, 0.f, 0.f};
    if (y >= 0 && y < V) {
      const uint2 wv = *(const uint2*)(W + y * H + c * 4);
      w[0] = __uint_as_float(wv.x << 16);
      w[1] = __uint_as_float(wv.x & 0xffff0000u);
      w[2] = __uint_as_float(wv.y << 16);
      w[3] = __uint_as_float(wv.y & 0xffff0000u);
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) s[e] = cf * (w[e] - scale * s[e]);
  }
  bf16x4 o;
#pragma unroll
  for (int e = 0; e < 4; ++e) o[e] = (__bf16)s[e];
  ((bf16x4*)out)[rows.token((int)r) * h4 + c] = o;
}

// ----------------------------------------------------------------------------
// Transpose and plain GEMM
// ----------------------------------------------------------------------------
__global__ __launch_bounds__(256) void transpose_bf16_kernel(const uint16_t* __restrict__ in,
                                                             uint16_t* __restrict__ out, int64_t R,
                                                             int64_t C) {
  __shared__ uint16_t tile[64][66];
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

struct GemmParams {
  const void* P;
  const void* Q;
  void* out;
  int64_t M, N, K;
  int MT, NT, out_f32;
};

template <int NI>
__device__ __forceinline__ void gemm_nt_store(const TileAcc<NI>& acc, const GemmParams& p, int mt, int nt) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int wm = wave_m<NI>(wave), wn = wave_n<NI>(wave);
  const int half = lane >> 5;
  if (!p.out_f32 && (p.M & 7) == 0 && (int64_t)(mt + 1) * TILE <= p.M) {
    // bf16 and all 256 rows inside: 16-byte stores (lanes l and l + 32 hold the same column and trade halves)
#pragma unroll
    for (int ni = 0; ni < NI; ++ni) {
      const int64_t col = (int64_t)nt * TILE + acc_col<NI>(wn, ni, lane);
      if (col >= p.N) continue;
#pragma unroll
      for (int mi = 0; mi < 4; ++mi)
        store_block_bf16((uint16_t*)p.out + col * p.M + (int64_t)mt * TILE + wm * 128 + mi * 32, acc.c[mi][ni], half);
    }
    return;
  }
#pragma unroll
  for (int ni = 0; ni < NI; ++ni) {
    const int64_t col = (int64_t)nt * TILE + acc_col<NI>(wn, ni, lane);
    if (col >= p.N) continue;
#pragma unroll
    for (int mi = 0; mi < 4; ++mi)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int64_t m = (int64_t)mt * TILE + wm * 128 + mi * 32 + q * 8 + half * 4;
        if (m >= p.M) continue;
        if (p.out_f32) {
          floatx4 o;
#pragma unroll
          for (int e = 0; e < 4; ++e) o[e] = acc.c[mi][ni][q * 4 + e];
          *(floatx4*)((float*)p.out + col * p.M + m) = o;
        } else {
          bf16x4 o;
#pragma unroll
          for (int e = 0; e < 4; ++e) o[e] = (__bf16)acc.c[mi][ni][q * 4 + e];
          *(bf16x4*)((uint16_t*)p.out + col * p.M + m) = o;
        }
      }
  }
}

// Persistent: one work-group per CU walks tiles b, b + grid, ...; the next tile's first DMA stage is started
// before the current tile is stored.
__global__ __launch_bounds__(nthreads<GEMM_NI>()) void gemm_nt_kernel(GemmParams p) {
  __shared__ __attribute__((aligned(1024))) char smem[GEMM_LDS_BYTES];
  const int n_tiles = p.MT * p.NT;
  const int group = p.MT >= 8 * p.NT ? TILE_GROUP_STREAMING : TILE_GROUP;
  int t = blockIdx.x, mt, nt;
  tile_coords(xcd_remap(t, n_tiles), p.MT, p.NT, mt, nt, group);
  {
    PlainTileLoaders first;
    first.init(p.P, p.K, (int64_t)mt * TILE, p.M, p.Q, p.K, (int64_t)nt * TILE, p.N, 0, (int)p.K);
    first.issue_first(smem);
  }
  for (;;) {
    const int t2 = t + gridDim.x;
    const bool more = t2 < n_tiles;
    int mt2 = 0, nt2 = 0;
    if (more) tile_coords(xcd_remap(t2, n_tiles), p.MT, p.NT, mt2, nt2, group);
    TileAcc<GEMM_NI> acc;
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
    gemm_nt_store<GEMM_NI>(acc, p, mt, nt);
    if (!more) break;
    t = t2;
    mt = mt2;
    nt = nt2;
  }
}

// ----------------------------------------------------------------------------
// Host side
// ----------------------------------------------------------------------------
static int num_cus() {
  static int n = 0;
  if (n == 0) {
    int dev = 0, v = 0;
    if (hipGetDevice(&dev) == hipSuccess &&
        hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0)
      n = v;
    else
      n = 256;
  }
  return n;
}

// Split count for the d_hidden GEMM: fill whole rounds of CUs, keep every split
// at least 32 K-steps long, prefer fewer splits on ties.
static int choose_nsplit(int tiles, int ksteps) {
  const int cus = num_cus();
  int best = 1;
  double best_eff = 0.0;
  for (int ns = 1; ns <= 16; ++ns) {
    if (ksteps / ns < 32 && ns > 1) break;
    int blocks = tiles * ns;
    int rounds = (blocks + cus - 1) / cus;
    double eff = (double)blocks / ((double)rounds * cus);
    if (eff > best_eff + 0.02) {
      best_eff = eff;
      best = ns;
    }
  }
  return best;
}

static int32_t check_common(const void* hidden, const void* lm_head, int64_t T, int64_t S,
                            int64_t V, int64_t H, bool need_v64) {
  ARTK_CHECK_ARG(hidden && lm_head, "null hidden or lm_head pointer");
  ARTK_CHECK_ARG(aligned16(hidden) && aligned16(lm_head), "hidden and lm_head must be 16-byte aligned");
  ARTK_CHECK_ARG(T > 0 && S > 0 && V > 0 && H > 0, "T, S, V, H must be positive");
  ARTK_CHECK_ARG(T % S == 0, "T (%lld) must be a multiple of the row length S (%lld)", (long long)T,
                 (long long)S);
  if (H % BK != 0) {
    set_error("hidden size %lld must be a multiple of %d", (long long)H, BK);
    return ARTK_ERR_UNSUPPORTED_SHAPE;
  }
  if (V % 8 != 0 || (need_v64 && V % BK != 0)) {
    set_error("vocab size %lld must be a multiple of %d", (long long)V, need_v64 ? BK : 8);
    return ARTK_ERR_UNSUPPORTED_SHAPE;
  }
  if (T >= (1ll << 31) / 4 || V >= (1ll << 31) / 512) {
    set_error("T or V too large");
    return ARTK_ERR_UNSUPPORTED_SHAPE;
  }
  return ARTK_OK;
}

static ChunkRows dense_rows(int64_t t0, int64_t n) {
  ChunkRows r;
  r.row_token = nullptr;
  r.n_all = nullptr;
  r.t0 = t0;
  r.c0 = 0;
  r.cap = (int)n;
  return r;
}

// Launch K0 (when the chunk is stashed), K1 (+ NaN pre-fill of sel) and K2 for the rows of one chunk.  `logprob`
// (may be null) is the whole batch's array; `lse_chunk` is indexed by chunk row.
static int32_t launch_fwd_chunk(const void* hidden, const void* lm_head, const int64_t* ids,
                                int shift, const ChunkRows& rows, int64_t S, int64_t V, int64_t H,
                                float2* part, float* sel, uint16_t* stash, float* ref, const uint8_t* need,
                                float* logprob, float* lse_chunk, hipStream_t st) {
  const int64_t Tc = rows.cap;
  if (stash) {
    prof_begin(PROF_TARGET_REF, st);
    target_ref_kernel<<<(unsigned)((Tc + 3) / 4), 256, 0, st>>>(
        (const uint16_t*)(rows.row_token ? hidden : (const void*)((const char*)hidden + rows.t0 * H * 2)),
        (const uint16_t*)lm_head, ids, rows, need, S, shift, V, H, ref);
    prof_end(PROF_TARGET_REF, st);
    ARTK_CHECK_LAUNCH();
  }
  FwdParams p;
  p.hidden = rows.row_token ? hidden : (const void*)((const char*)hidden + rows.t0 * H * 2);
  p.W = lm_head;
  p.ids = ids;
  p.rows = rows;
  p.Tc = Tc;
  p.S = S;
  p.V = V;
  p.H = H;
  p.shift = shift;
  p.part = part;
  p.sel = sel;
  p.stash = stash;
  p.ref = ref;
  p.need = need;
  p.VT = (int)((V + TILE - 1) / TILE);
  p.TT = (int)((Tc + TILE - 1) / TILE);
  fill_f32_kernel<<<(unsigned)((Tc + 255) / 256), 256, 0, st>>>(sel, Tc, NAN);
  ARTK_CHECK_LAUNCH();
  const int n_tiles = p.VT * p.TT;
  const unsigned grid = (unsigned)(n_tiles < num_cus() ? n_tiles : num_cus());
  prof_begin(PROF_LMHEAD_FWD, st);
  const bool gather = rows.row_token != nullptr;
  if (stash && gather)
    lmhead_fwd_kernel<true, true><<<grid, nthreads<FWD_NI>(), 0, st>>>(p);
  else if (stash)
    lmhead_fwd_kernel<true, false><<<grid, nthreads<FWD_NI>(), 0, st>>>(p);
  else if (gather)
    lmhead_fwd_kernel<false, true><<<grid, nthreads<FWD_NI>(), 0, st>>>(p);
  else
    lmhead_fwd_kernel<false, false><<<grid, nthreads<FWD_NI>(), 0, st>>>(p);
  prof_end(PROF_LMHEAD_FWD, st);
  ARTK_CHECK_LAUNCH();
  lse_finalize_kernel<<<(unsigned)((Tc + 15) / 16), 256, 0, st>>>(part, 2 * p.VT, Tc, rows, sel, logprob,
                                                                    lse_chunk);
  ARTK_CHECK_LAUNCH();
  return ARTK_OK;
}

// fp32 partial rows of the d_hidden GEMM for a chunk of Tc rows: enough for the
// split count the dense case would use.
static int64_t bwd_part_rows(int64_t Tc, int64_t H, int64_t V) {
  const int64_t tt = (Tc + TILE - 1) / TILE;
  const int tiles = (int)(((H + TILE - 1) / TILE) * tt);
  return (int64_t)choose_nsplit(tiles, (int)(V / BK)) * tt * TILE;
}

struct BwdScratch {
  float* partial;
  int64_t part_rows;
  int* active_idx;
  int* pos;
  int* sched;
};

// Launch K3a, K4, K5 for one chunk whose exponentials (see target_ref_kernel) are in `stash`.
// `d_hidden` is the whole batch's gradient, indexed by position.
static int32_t launch_bwd_chunk(uint16_t* stash, const void* lm_head, const void* lm_head_t, const int64_t* ids,
                                int shift, const ChunkRows& rows, int64_t S, int64_t V, int64_t H,
                                const float* lse_chunk, const float* coef_chunk, const float* ref_chunk,
                                const BwdScratch& sc, uint16_t* d_hidden, int* dropped, hipStream_t st) {
  const int64_t Tc = rows.cap;
  const int HT = (int)((H + TILE - 1) / TILE);
  const int TT = (int)((Tc + TILE - 1) / TILE);
  compact_rows_kernel<<<1, 1024, 0, st>>>(coef_chunk, rows, HT, (int)(V / BK), (int)sc.part_rows,
                                          num_cus(), sc.active_idx, sc.pos, sc.sched);
  ARTK_CHECK_LAUNCH();
  BwdParams b;
  b.Wt = lm_head_t;
  b.P = stash;
  b.V = V;
  b.H = H;
  b.HT = HT;
  b.active_idx = sc.active_idx;
  b.sched = sc.sched;
  b.partial = sc.partial;
  const int64_t max_blocks = sc.part_rows / TILE * HT;  // tiles * splits can never exceed this
  const int64_t dense_cap = (int64_t)HT * TT * 16;
  const unsigned grid = (unsigned)(max_blocks < dense_cap ? max_blocks : dense_cap);
  prof_begin(PROF_DHIDDEN_GEMM, st);
  dhidden_gemm_kernel<<<grid, nthreads<BWD_NI>(), 0, st>>>(b);
  prof_end(PROF_DHIDDEN_GEMM, st);
  ARTK_CHECK_LAUNCH();
  const int64_t n4 = Tc * H / 4;
  splitk_reduce_kernel<<<(unsigned)((n4 + 255) / 256), 256, 0, st>>>(
      sc.partial, sc.pos, sc.sched, rows, H, V, coef_chunk, lse_chunk, ref_chunk, ids, S, shift,
      (const uint16_t*)lm_head, d_hidden, dropped);
  ARTK_CHECK_LAUNCH();
  return ARTK_OK;
}

// ----------------------------------------------------------------------------
// Scratch of artk_grpo_loss_static: a device array that is part of the code
// object, so the entry point needs no allocation.  Every GPU the library runs on
// holds its own copy at its own address; the array's name is only a handle for
// hipGetSymbolAddress on the host, never a device pointer.
// ----------------------------------------------------------------------------
constexpr size_t STATIC_SCRATCH_BYTES =
    2 * ((size_t)ARTK_GRPO_LOSS_STATIC_MAX_T * sizeof(float) + 256) + 64 * sizeof(int) + 512;
static __device__ __align__(256) unsigned char scratch[STATIC_SCRATCH_BYTES];

constexpr int STATIC_MAX_DEVICES = 64;
static void* g_scratch_ptr[STATIC_MAX_DEVICES];  // device address of `scratch` per device, once resolved
static std::mutex g_scratch_mu;

// Device address of `scratch` on the current device (resolved on the first call per device).
static int32_t static_scratch_base(void** out) {
  int dev = -1;
  ARTK_CHECK_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= STATIC_MAX_DEVICES) {
    set_error("device ordinal %d outside [0, %d)", dev, STATIC_MAX_DEVICES);
    return ARTK_ERR_UNSUPPORTED_SHAPE;
  }
  std::lock_guard<std::mutex> lk(g_scratch_mu);
  if (g_scratch_ptr[dev] == nullptr) {
    void* ptr = nullptr;
    ARTK_CHECK_HIP(hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch)));
    if (ptr == nullptr) {
      set_error("hipGetSymbolAddress returned a null address for the static scratch");
      return ARTK_ERR_INVALID_ARGUMENT;
    }
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return ARTK_OK;
}

}  // namespace artk

using namespace artk;

extern "C" {

size_t artk_logprob_fwd_workspace_bytes(int64_t T, int64_t V, int64_t H) {
  (void)H;
  Workspace ws(nullptr, 0);
  int64_t VT = (V + TILE - 1) / TILE;
  ws.take<float2>((size_t)(2 * VT * T));
  ws.take<float>((size_t)T);
  return ws.used + 256;
}

int32_t artk_logprob_fwd(const void* hidden, const void* lm_head, const int64_t* ids, int32_t shift,
                         int64_t T, int64_t S, int64_t V, int64_t H, float* logprob, float* lse,
                         void* workspace, size_t workspace_bytes, artk_stream_t stream) {
  int32_t rc = check_common(hidden, lm_head, T, S, V, H, false);
  if (rc) return rc;
  ARTK_CHECK_ARG(ids && logprob && lse, "null ids/logprob/lse pointer");
  ARTK_CHECK_ARG(shift == 0 || shift == 1, "shift must be 0 or 1");
  Workspace ws(workspace, workspace_bytes);
  int64_t VT = (V + TILE - 1) / TILE;
  float2* part = ws.take<float2>((size_t)(2 * VT * T));
  float* sel = ws.take<float>((size_t)T);
  if (!ws.ok()) {
    set_error("workspace too small: need %zu bytes, got %zu", ws.used, workspace_bytes);
    return ARTK_ERR_WORKSPACE_TOO_SMALL;
  }
  return launch_fwd_chunk(hidden, lm_head, ids, shift, dense_rows(0, T), S, V, H, part, sel, nullptr, nullptr,
                          nullptr, logprob, lse, (hipStream_t)stream);
}

// Scratch of one chunk of Tc positions carved out of the caller's workspace.
struct ChunkScratch {
  uint16_t* stash;  // [Tc,V] bf16 exp(logit - ref) of the rows the backward reads
  float2* part;     // [2*VT][Tc]
  float* sel;       // [Tc]
  float* ref;       // [Tc] reference logit per chunk row (target_ref_kernel)
  uint8_t* need;    // [Tc]
  BwdScratch bwd;
  float *lse, *coef;            // [Tc] each, by chunk row (fused op only)
  float *pl, *kl;               // [T] each, by position (fused op only)
  int* count;
  int* eval_idx;                // [T] positions the forward is evaluated for (fused op, skip mode)
  int* n_eval;
  float* lse_tmp;               // [Tc] (standalone backward only)
};

static void carve(Workspace& ws, int64_t T, int64_t V, int64_t H, int64_t Tc, bool fused,
                  ChunkScratch& c) {
  const int64_t VT = (V + TILE - 1) / TILE;
  c.stash = ws.take<uint16_t>((size_t)(Tc * V));
  c.part = ws.take<float2>((size_t)(2 * VT * Tc));
  c.sel = ws.take<float>((size_t)Tc);
  c.ref = ws.take<float>((size_t)Tc);
  c.need = ws.take<uint8_t>((size_t)Tc);
  c.bwd.part_rows = bwd_part_rows(Tc, H, V);
  c.bwd.partial = ws.take<float>((size_t)c.bwd.part_rows * H);
  c.bwd.active_idx = ws.take<int>((size_t)Tc);
  c.bwd.pos = ws.take<int>((size_t)Tc);
  c.bwd.sched = ws.take<int>(64);
  if (fused) {
    c.lse = ws.take<float>((size_t)Tc);
    c.coef = ws.take<float>((size_t)Tc);
    c.pl = ws.take<float>((size_t)T);
    c.kl = ws.take<float>((size_t)T);
    c.count = ws.take<int>(64);
    c.eval_idx = ws.take<int>((size_t)T);
    c.n_eval = ws.take<int>(64);
  } else {
    c.lse_tmp = ws.take<float>((size_t)Tc);
  }
}

// Chunk length: the caller's wish (<= 0: automatic, about 6000 positions split
// evenly), at most T, and small enough that a row offset inside the logits
// scratch fits the 31-bit offsets of the GEMM loader.
static int64_t clamp_chunk(int64_t T, int64_t V, int64_t chunk_tokens) {
  int64_t cap = ((1ll << 30) - 1) / V / TILE * TILE;  // Tc * V * 2 bytes < 2^31
  if (cap < TILE) cap = TILE;
  if (chunk_tokens <= 0) {
    const int64_t want = cap < 6144 ? cap : 6144;
    const int64_t n = (T + want - 1) / want;
    chunk_tokens = ((T + n - 1) / n + TILE - 1) / TILE * TILE;
  }
  if (chunk_tokens > cap) chunk_tokens = cap;
  if (chunk_tokens > T) chunk_tokens = T;
  return chunk_tokens;
}

// Lengths of the chunks of a batch of T positions with at most Tc per chunk.  When Tc is
// a whole number of tiles the tiles are spread evenly over the chunks (16384 positions, Tc
// = 5632: 22 + 21 + 21 tiles rather than 22 + 22 + 20), which wastes less of the last round
// of work-groups of each forward launch.
struct ChunkSteps {
  int64_t Tc, base, extra;
  bool balanced;
  ChunkSteps(int64_t T, int64_t Tc_, bool allow) : Tc(Tc_), base(0), extra(0), balanced(false) {
    if (allow && Tc % TILE == 0) {
      const int64_t nchunks = (T + Tc - 1) / Tc, tiles = (T + TILE - 1) / TILE;
      base = tiles / nchunks;
      extra = tiles % nchunks;
      balanced = true;
    }
  }
  int64_t step(int64_t chunk) const { return balanced ? (base + (chunk < extra ? 1 : 0)) * TILE : Tc; }
};

size_t artk_logprob_bwd_workspace_bytes(int64_t T, int64_t V, int64_t H, int64_t chunk_tokens) {
  Workspace ws(nullptr, 0);
  ChunkScratch c;
  carve(ws, T, V, H, clamp_chunk(T, V, chunk_tokens), false, c);
  return ws.used + 256;
}

int32_t artk_logprob_bwd(const void* hidden, const void* lm_head, const void* lm_head_t,
                         const int64_t* ids, int32_t shift, int64_t T, int64_t S, int64_t V,
                         int64_t H, const float* lse, const float* grad_logprob, void* d_hidden,
                         int64_t chunk_tokens, void* workspace, size_t workspace_bytes,
                         artk_stream_t stream) {
  int32_t rc = check_common(hidden, lm_head, T, S, V, H, true);
  if (rc) return rc;
  ARTK_CHECK_ARG(lm_head_t && ids && lse && grad_logprob && d_hidden, "null pointer argument");
  ARTK_CHECK_ARG(aligned16(lm_head_t) && aligned16(d_hidden), "pointers must be 16-byte aligned");
  ARTK_CHECK_ARG(shift == 0 || shift == 1, "shift must be 0 or 1");
  const int64_t Tc = clamp_chunk(T, V, chunk_tokens);
  Workspace ws(workspace, workspace_bytes);
  ChunkScratch c;
  carve(ws, T, V, H, Tc, false, c);
  if (!ws.ok()) {
    set_error("workspace too small: need %zu bytes, got %zu", ws.used, workspace_bytes);
    return ARTK_ERR_WORKSPACE_TOO_SMALL;
  }
  hipStream_t st = (hipStream_t)stream;
  const ChunkSteps steps(T, Tc, true);
  int64_t step = 0;
  for (int64_t t0 = 0, ci = 0; t0 < T; t0 += step, ++ci) {
    step = steps.step(ci);
    const int64_t n = (T - t0 < step) ? (T - t0) : step;
    // The scratch row pitch is V, so a shorter chunk simply uses fewer rows.
    need_from_grad_kernel<<<(unsigned)((n + 255) / 256), 256, 0, st>>>(grad_logprob + t0, n, c.need);
    ARTK_CHECK_LAUNCH();
    const ChunkRows rows = dense_rows(t0, n);
    rc = launch_fwd_chunk(hidden, lm_head, ids, shift, rows, S, V, H, c.part, c.sel, c.stash, c.ref, c.need,
                          nullptr, c.lse_tmp, st);
    if (rc) return rc;
    rc = launch_bwd_chunk(c.stash, lm_head, lm_head_t, ids, shift, rows, S, V, H, lse + t0, grad_logprob + t0,
                          c.ref, c.bwd, (uint16_t*)d_hidden, nullptr, st);
    if (rc) return rc;
  }
  return ARTK_OK;
}

size_t artk_grpo_loss_workspace_bytes(int64_t T) {
  Workspace ws(nullptr, 0);
  ws.take<float>((size_t)T);
  ws.take<float>((size_t)T);
  ws.take<int>(64);
  return ws.used + 256;
}

// Shared body of artk_grpo_loss and artk_grpo_loss_static: the scratch (two f32 [T]
// arrays of per-token terms and the mask count) is carved out of `ws`.
static int32_t grpo_loss_run(const float* new_logprob, const float* old_logprob, const float* advantages,
                             const uint8_t* mask, const float* weights, const float* ref_logprob,
                             int32_t shift, int64_t T, int64_t S, float clip_lo, float clip_hi, float beta,
                             float* scalars, float* coef, Workspace& ws, hipStream_t st) {
  ARTK_CHECK_ARG(new_logprob && old_logprob && advantages && mask && weights && scalars,
                 "null pointer argument");
  ARTK_CHECK_ARG(T > 0 && S > 0 && T % S == 0 && T < (1ll << 31), "T must be a positive multiple of S below 2^31");
  ARTK_CHECK_ARG(shift == 0 || shift == 1, "shift must be 0 or 1");
  ARTK_CHECK_ARG(clip_lo <= clip_hi, "clip_lo must not exceed clip_hi");
  float* pl = ws.take<float>((size_t)T);
  float* kl = ws.take<float>((size_t)T);
  int* count = ws.take<int>(64);
  if (!ws.ok()) {
    set_error("workspace too small: need %zu bytes, got %zu", ws.used, ws.size);
    return ARTK_ERR_WORKSPACE_TOO_SMALL;
  }
  mask_count_kernel<<<1, 1024, 0, st>>>(mask, T, S, shift, count);
  ARTK_CHECK_LAUNCH();
  LossParams p;
  p.new_lp = new_logprob;
  p.old_lp = old_logprob;
  p.adv = advantages;
  p.mask = mask;
  p.weights = weights;
  p.ref_lp = (beta > 0.f) ? ref_logprob : nullptr;
  p.count = count;
  p.rows = dense_rows(0, T);
  p.S = S;
  p.shift = shift;
  p.clip_lo = clip_lo;
  p.clip_hi = clip_hi;
  p.beta = beta;
  p.pl_tok = pl;
  p.kl_tok = kl;
  p.coef = coef;
  grpo_loss_tok_kernel<<<(unsigned)((T + 255) / 256), 256, 0, st>>>(p);
  ARTK_CHECK_LAUNCH();
  grpo_loss_reduce_kernel<<<1, 1024, 0, st>>>(pl, kl, T, count, p.ref_lp ? beta : 0.f, 0, scalars);
  ARTK_CHECK_LAUNCH();
  return ARTK_OK;
}

int32_t artk_grpo_loss(const float* new_logprob, const float* old_logprob, const float* advantages,
                       const uint8_t* mask, const float* weights, const float* ref_logprob,
                       int32_t shift, int64_t T, int64_t S, float clip_lo, float clip_hi, float beta,
                       float* scalars, float* coef, void* workspace, size_t workspace_bytes,
                       artk_stream_t stream) {
  Workspace ws(workspace, workspace_bytes);
  return grpo_loss_run(new_logprob, old_logprob, advantages, mask, weights, ref_logprob, shift, T, S,
                       clip_lo, clip_hi, beta, scalars, coef, ws, (hipStream_t)stream);
}

int32_t artk_grpo_loss_static(const float* new_logprob, const float* old_logprob, const float* advantages,
                              const uint8_t* mask, const float* weights, const float* ref_logprob,
                              int32_t shift, int64_t T, int64_t S, float clip_lo, float clip_hi,
                              float beta, float* scalars, float* coef, artk_stream_t stream) {
  if (T > ARTK_GRPO_LOSS_STATIC_MAX_T) {
    set_error("artk_grpo_loss_static handles at most %d positions per call, got %lld (use artk_grpo_loss "
              "with a caller-provided workspace)",
              ARTK_GRPO_LOSS_STATIC_MAX_T, (long long)T);
    return ARTK_ERR_UNSUPPORTED_SHAPE;
  }
  void* base = nullptr;
  const int32_t rc = static_scratch_base(&base);
  if (rc) return rc;
  Workspace ws(base, STATIC_SCRATCH_BYTES);
  return grpo_loss_run(new_logprob, old_logprob, advantages, mask, weights, ref_logprob, shift, T, S,
                       clip_lo, clip_hi, beta, scalars, coef, ws, (hipStream_t)stream);
}

size_t artk_grpo_fused_workspace_bytes(int64_t T, int64_t V, int64_t H, int64_t chunk_tokens) {
  Workspace ws(nullptr, 0);
  ChunkScratch c;
  carve(ws, T, V, H, clamp_chunk(T, V, chunk_tokens), true, c);
  return ws.used + 256;
}

int32_t artk_grpo_fused(const void* hidden, const void* lm_head, const void* lm_head_t,
                        const int64_t* tokens, const float* old_logprob, const float* advantages,
                        const uint8_t* mask, const float* weights, const float* ref_logprob,
                        int64_t T, int64_t S, int64_t V, int64_t H, float clip_lo, float clip_hi,
                        float beta, int64_t chunk_tokens, int32_t flags, float* scalars,
                        float* logprob, void* d_hidden, void* workspace, size_t workspace_bytes,
                        artk_stream_t stream) {
  int32_t rc = check_common(hidden, lm_head, T, S, V, H, true);
  if (rc) return rc;
  ARTK_CHECK_ARG(lm_head_t && tokens && old_logprob && advantages && mask && weights && scalars &&
                     logprob && d_hidden,
                 "null pointer argument");
  ARTK_CHECK_ARG(aligned16(lm_head_t) && aligned16(d_hidden), "pointers must be 16-byte aligned");
  ARTK_CHECK_ARG(clip_lo <= clip_hi, "clip_lo must not exceed clip_hi");
  ARTK_CHECK_ARG((flags & ~ARTK_FUSED_SKIP_INACTIVE) == 0, "unknown flag bits 0x%x", (unsigned)flags);
  const bool skip = (flags & ARTK_FUSED_SKIP_INACTIVE) != 0;
  if (skip && T * H * 2 >= (1ll << 31)) {
    // gathered rows of `hidden` are addressed with 31-bit byte offsets
    set_error("ARTK_FUSED_SKIP_INACTIVE needs T*H*2 < 2^31 bytes of hidden states");
    return ARTK_ERR_UNSUPPORTED_SHAPE;
  }
  const int64_t Tc = clamp_chunk(T, V, chunk_tokens);
  Workspace ws(workspace, workspace_bytes);
  ChunkScratch c;
  carve(ws, T, V, H, Tc, true, c);
  if (!ws.ok()) {
    set_error("workspace too small: need %zu bytes, got %zu", ws.used, workspace_bytes);
    return ARTK_ERR_WORKSPACE_TOO_SMALL;
  }
  hipStream_t st = (hipStream_t)stream;
  const float* ref = (beta > 0.f) ? ref_logprob : nullptr;
  mask_count_kernel<<<1, 1024, 0, st>>>(mask, T, S, 1, c.count);
  ARTK_CHECK_LAUNCH();
  if (skip) {
    // Positions that are not evaluated keep: logprob NaN, zero loss terms, zero d_hidden.
    compact_eval_kernel<<<1, 1024, 0, st>>>(mask, weights, advantages, ref, T, S, 1, c.eval_idx,
                                            c.n_eval);
    ARTK_CHECK_LAUNCH();
    const unsigned gT = (unsigned)((T + 255) / 256);
    fill_f32_kernel<<<gT, 256, 0, st>>>(logprob, T, NAN);
    ARTK_CHECK_LAUNCH();
    fill_f32_kernel<<<gT, 256, 0, st>>>(c.pl, T, 0.f);
    ARTK_CHECK_LAUNCH();
    fill_f32_kernel<<<gT, 256, 0, st>>>(c.kl, T, 0.f);
    ARTK_CHECK_LAUNCH();
    const int64_t nd = T * H / 2;  // bf16 pairs
    fill_f32_kernel<<<(unsigned)((nd + 255) / 256), 256, 0, st>>>((float*)d_hidden, nd, 0.f);
    ARTK_CHECK_LAUNCH();
  }
  // In skip mode the number of evaluated rows is known only on the device: every
  // chunk the worst case needs is launched and the ones past the end do nothing.
  const ChunkSteps steps(T, Tc, !skip);
  int64_t step = 0;
  for (int64_t t0 = 0, ci = 0; t0 < T; t0 += step, ++ci) {
    step = steps.step(ci);
    ChunkRows rows;
    if (skip) {
      rows.row_token = c.eval_idx + t0;
      rows.n_all = c.n_eval;
      rows.t0 = 0;
      rows.c0 = (int)t0;
      rows.cap = (int)Tc;
    } else {
      const int64_t n = (T - t0 < step) ? (T - t0) : step;
      rows = dense_rows(t0, n);
      need_from_inputs_kernel<<<(unsigned)((n + 255) / 256), 256, 0, st>>>(mask, weights, advantages,
                                                                           ref, t0, n, S, 1, c.need);
      ARTK_CHECK_LAUNCH();
    }
    rc = launch_fwd_chunk(hidden, lm_head, tokens, 1, rows, S, V, H, c.part, c.sel, c.stash, c.ref,
                          skip ? nullptr : c.need, logprob, c.lse, st);
    if (rc) return rc;
    LossParams p;
    p.new_lp = logprob;
    p.old_lp = old_logprob;
    p.adv = advantages;
    p.mask = mask;
    p.weights = weights;
    p.ref_lp = ref;
    p.count = c.count;
    p.rows = rows;
    p.S = S;
    p.shift = 1;
    p.clip_lo = clip_lo;
    p.clip_hi = clip_hi;
    p.beta = beta;
    p.pl_tok = c.pl;
    p.kl_tok = c.kl;
    p.coef = c.coef;
    grpo_loss_tok_kernel<<<(unsigned)((rows.cap + 255) / 256), 256, 0, st>>>(p);
    ARTK_CHECK_LAUNCH();
    rc = launch_bwd_chunk(c.stash, lm_head, lm_head_t, tokens, 1, rows, S, V, H, c.lse, c.coef, c.ref, c.bwd,
                          (uint16_t*)d_hidden, c.count + 1, st);
    if (rc) return rc;
  }
  grpo_loss_reduce_kernel<<<1, 1024, 0, st>>>(c.pl, c.kl, T, c.count, ref ? beta : 0.f, 1, scalars);
  ARTK_CHECK_LAUNCH();
  return ARTK_OK;
}

int32_t artk_transpose_bf16(const void* in, void* out, int64_t R, int64_t C, artk_stream_t stream) {
  ARTK_CHECK_ARG(in && out, "null pointer argument");
  ARTK_CHECK_ARG(R > 0 && C > 0, "R and C must be positive");
  dim3 grid((unsigned)((C + 63) / 64), (unsigned)((R + 63) / 64));
  transpose_bf16_kernel<<<grid, 256, 0, (hipStream_t)stream>>>((const uint16_t*)in, (uint16_t*)out, R,
                                                               C);
  ARTK_CHECK_LAUNCH();
  return ARTK_OK;
}

int32_t artk_gemm_nt(const void* P, const void* Q, void* out, int64_t M, int64_t N, int64_t K,
                     int32_t out_f32, artk_stream_t stream) {
  ARTK_CHECK_ARG(P && Q && out, "null pointer argument");
  ARTK_CHECK_ARG(aligned16(P) && aligned16(Q) && aligned16(out), "pointers must be 16-byte aligned");
  ARTK_CHECK_ARG(M > 0 && N > 0 && K > 0, "M, N, K must be positive");
  if (K % BK != 0 || M % 4 != 0) {
    set_error("K must be a multiple of %d and M a multiple of 4", BK);
    return ARTK_ERR_UNSUPPORTED_SHAPE;
  }
  GemmParams p;
  p.P = P;
  p.Q = Q;
  p.out = out;
  p.M = M;
  p.N = N;
  p.K = K;
  p.MT = (int)((M + TILE - 1) / TILE);
  p.NT = (int)((N + TILE - 1) / TILE);
  p.out_f32 = out_f32;
  const int64_t n_tiles = (int64_t)p.MT * p.NT;
  gemm_nt_kernel<<<(unsigned)(n_tiles < num_cus() ? n_tiles : num_cus()), nthreads<GEMM_NI>(), 0, (hipStream_t)stream>>>(p);
  ARTK_CHECK_LAUNCH();
  return ARTK_OK;
}

}  // extern "C"
