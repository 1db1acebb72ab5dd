// Packed-row attention for gfx950 (MI355X, CDNA4).
//
// The reference materialises a dense [1,S,S] additive bias from the packed
// row's ids (src/art/local/train.py:177-215):
//     visible(i, j) = j <= i && (group[i] == group[j] || parent[i] == group[j])
// and passes it to the model as `causal_mask` (train.py:239-241).  Here the
// matrix is never built.  A plan (once per packed row, shared by every layer
// and head) turns the 64-bit ids into int32 equality codes and classifies each
// (query block, key block) pair as invisible / partly visible / fully visible;
// the attention kernels walk only the visible blocks and evaluate the rule per
// element only in the partly visible ones.
//
// Forward work-group: 256 queries x one head, 8 wavefronts of 32 queries, key
// tiles of 64.  Scores are computed transposed (S^T = K Q^T, MFMA 32x32x16), so
// that a lane owns one query: the row maximum and sum are in-lane reductions
// plus one exchange between the two half-waves, the accumulator of S^T is
// already in the B-operand layout of the second product O^T = V^T P^T, and the
// running rescale of O^T is a per-lane scalar.  K tiles ([key][d]) and V^T
// tiles ([d][key], from a transposed copy of V made once per call) are brought
// into a 3-stage LDS ring by buffer_load ... lds.
#include <stdlib.h>

#include "common.hpp"
#include "gemm_nt.hpp"

namespace artk {

constexpr int ATT_BM = 256;    // queries per work-group
constexpr int ATT_BN = 64;     // keys per tile
constexpr int ATT_STAGES = 3;
constexpr float ATT_LAZY = 8.f;   // forward: how far a score may exceed the exponentials' reference (log2 units)
constexpr int ATT_MAX_KB = 1024;  // key blocks per row the list in LDS can hold
constexpr int ATT_BQ2 = 64;    // dK/dV kernel: queries per tile
constexpr int ATT_BK2 = 128;   // dK/dV kernel: keys per work-group (4 key groups x 32)
// dK/dV with grouped-query heads: a key block seen by at most this many (query
// tile, head) pairs is handled by ONE work-group for all heads of its group (no
// partial sums); busier blocks get one work-group per head.
constexpr int ATT_LIGHT_MAX = 64;

// ----------------------------------------------------------------------------
// Plan
// ----------------------------------------------------------------------------

// gc[t] = first position whose group id equals group_ids[t];
// pc[t] = first position whose group id equals parent_ids[t], or -2 if none.
// Then group[i] == group[j] <=> gc[i] == gc[j] and parent[i] == group[j] <=>
// pc[i] == gc[j].  Brute force over all pairs (integer work, once per row).
__global__ __launch_bounds__(256) void attn_codes_kernel(const int64_t* __restrict__ group_ids,
                                                         const int64_t* __restrict__ parent_ids,
                                                         int S, int* __restrict__ gc,
                                                         int* __restrict__ pc) {
  __shared__ int64_t tile[256];
  const int t = blockIdx.x * 256 + threadIdx.x;
  const int64_t g = t < S ? group_ids[t] : 0;
  const int64_t pa = t < S ? parent_ids[t] : 0;
  int first_g = 0x7fffffff, first_p = 0x7fffffff;
  for (int j0 = 0; j0 < S; j0 += 256) {
    __syncthreads();
    tile[threadIdx.x] = j0 + (int)threadIdx.x < S ? group_ids[j0 + threadIdx.x] : 0;
    __syncthreads();
    const int lim = S - j0 < 256 ? S - j0 : 256;
    for (int jj = 0; jj < lim; ++jj) {
      const int64_t id = tile[jj];
      if (id == g && j0 + jj < first_g) first_g = j0 + jj;
      if (id == pa && j0 + jj < first_p) first_p = j0 + jj;
    }
  }
  if (t < S) {
    gc[t] = first_g;
    pc[t] = first_p == 0x7fffffff ? -2 : first_p;
  }
}

__device__ __forceinline__ bool attn_visible(int i, int j, int gi, int pi, int gj) {
  return j <= i && (gj == gi || gj == pi);
}

// Visibility of one (owner block, tile) pair, per wavefront of the kernel that
// will process it:
//   bits 14-15  1 = some pairs visible, 2 = all
//   bits 16-23  wave w has at least one visible pair in its part of the tile
//   bits 24-31  every pair of wave w's part is visible (no per-element test needed)
// 0 when nothing is visible.
// MODE 0 (forward, dQ): owner = 256 queries, tile = 64 keys, wave w = queries 32w..32w+31.
// MODE 1 (dK/dV):      owner = 128 keys, tile = 64 queries, wave w = keys 32(w&3).. x
//                      queries 32(w>>2)..
// One wavefront evaluates the rule on every pair of its (owner, tile).
template <int MODE>
__global__ __launch_bounds__(256) void attn_classify_kernel(const int* __restrict__ gc,
                                                            const int* __restrict__ pc, int n_tile,
                                                            uint32_t* __restrict__ info) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int tile = blockIdx.x * 4 + wave;
  const int owner = blockIdx.y;
  if (tile >= n_tile) return;
  uint32_t any = 0, all = 0;
  if (MODE == 0) {
    const int q0 = owner * ATT_BM, j = tile * ATT_BN + lane;
    if (tile * ATT_BN <= q0 + ATT_BM - 1) {
      const int gj = gc[j];
      for (int g = 0; g < 8; ++g) {
        int cnt = 0;
        for (int ii = 0; ii < 32; ++ii) {
          const int i = q0 + 32 * g + ii;
          cnt += attn_visible(i, j, gc[i], pc[i], gj) ? 1 : 0;
        }
        any |= (uint32_t)(__ballot(cnt > 0) != 0ull) << g;
        all |= (uint32_t)(__ballot(cnt == 32) == ~0ull) << g;
      }
    }
  } else {
    const int k0 = owner * ATT_BK2, q0 = tile * ATT_BQ2;
    if (k0 <= q0 + ATT_BQ2 - 1) {
      for (int iter = 0; iter < 2; ++iter) {
        const int j = k0 + 64 * iter + lane;
        const int gj = gc[j];
        for (int qh = 0; qh < 2; ++qh) {
          int cnt = 0;
          for (int ii = 0; ii < 32; ++ii) {
            const int i = q0 + 32 * qh + ii;
            cnt += attn_visible(i, j, gc[i], pc[i], gj) ? 1 : 0;
          }
          const unsigned long long ab = __ballot(cnt > 0), fb = __ballot(cnt == 32);
          for (int hh = 0; hh < 2; ++hh) {
            const int bit = 2 * iter + hh + 4 * qh;
            any |= (uint32_t)((uint32_t)(ab >> (32 * hh)) != 0u) << bit;
            all |= (uint32_t)((uint32_t)(fb >> (32 * hh)) == 0xffffffffu) << bit;
          }
        }
      }
    }
  }
  if (lane == 0) {
    const uint32_t cls = all == 0xffu ? 2u : 1u;
    info[(int64_t)owner * n_tile + tile] = any ? (cls << 14) | (any << 16) | (all << 24) : 0u;
  }
}

// list[row][0..cnt[row]) = tile index | info for the tiles of info[row][*] that
// are not 0, ascending.  One work-group per row.
__global__ __launch_bounds__(256) void attn_compact_kernel(const uint32_t* __restrict__ info, int ncol,
                                                           uint32_t* __restrict__ list,
                                                           int* __restrict__ cnt) {
  __shared__ int wtot[4];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int row = blockIdx.x;
  int base = 0;
  for (int c0 = 0; c0 < ncol; c0 += 256) {
    const int c = c0 + threadIdx.x;
    const uint32_t v = c < ncol ? info[(int64_t)row * ncol + c] : 0u;
    const unsigned long long m = __ballot(v != 0);
    const int rank = __popcll(m & ((1ull << lane) - 1ull));
    __syncthreads();
    if (lane == 0) wtot[wave] = __popcll(m);
    __syncthreads();
    int off = base;
    for (int w = 0; w < wave; ++w) off += wtot[w];
    if (v) list[(int64_t)row * ncol + off + rank] = (uint32_t)c | v;
    base += wtot[0] + wtot[1] + wtot[2] + wtot[3];
  }
  if (threadIdx.x == 0) cnt[row] = base;
}

// Device-memory layout of a plan for a row of S positions (S % 256 == 0).
struct AttnPlan {
  int* gc;
  int* pc;
  int nQb, nKb;        // forward / dQ: query blocks of 256, key tiles of 64
  uint32_t* info;      // [nQb][nKb]
  uint32_t* list;      // [nQb][nKb]
  int* cnt;            // [nQb]
  int nQb2, nKb2;      // dK/dV: key blocks of 128, query tiles of 64
  uint32_t* info2;     // [nKb2][nQb2]
  uint32_t* list2;     // [nKb2][nQb2]
  int* cnt2;           // [nKb2]
};

static size_t attn_plan_layout(void* base, size_t bytes, int64_t S, AttnPlan& pl) {
  Workspace ws(base, bytes);
  pl.nQb = (int)(S / ATT_BM);
  pl.nKb = (int)(S / ATT_BN);
  pl.nQb2 = (int)(S / ATT_BQ2);
  pl.nKb2 = (int)(S / ATT_BK2);
  pl.gc = ws.take<int>((size_t)S);
  pl.pc = ws.take<int>((size_t)S);
  pl.info = ws.take<uint32_t>((size_t)pl.nQb * pl.nKb);
  pl.list = ws.take<uint32_t>((size_t)pl.nQb * pl.nKb);
  pl.cnt = ws.take<int>((size_t)pl.nQb);
  pl.info2 = ws.take<uint32_t>((size_t)pl.nQb2 * pl.nKb2);
  pl.list2 = ws.take<uint32_t>((size_t)pl.nQb2 * pl.nKb2);
  pl.cnt2 = ws.take<int>((size_t)pl.nKb2);
  return ws.ok() || base == nullptr ? ws.used : (size_t)-1;
}

// ----------------------------------------------------------------------------
// Tiles and fragments shared by the three kernels
// ----------------------------------------------------------------------------
// Every operand tile in LDS is 64 rows (keys or queries) x D elements, row-major
// as in HBM, its 16-byte chunks XOR-swizzled by row.  Two ways to read it:
//   row fragments  (ds_read_b128): lane (m, h) gets 8 consecutive d of row m,
//                   the A operand of a product that contracts over d;
//   transposed fragments (ds_read_b64_tr_b16, a gfx950 instruction): lane (m, h)
//                   gets element d = m of 8 rows, the A operand of a product
//                   that contracts over the tile's rows.  No transposed copies
//                   of K, V, Q or dO exist anywhere.
template <int D>
struct AttnTile {
  static constexpr int CHK = D / 8;                    // 16-byte chunks of a row
  static constexpr int ROW = D * 2;                    // bytes
  static constexpr int BYTES = 64 * ROW;
  static constexpr int N8 = BYTES / 1024 / 8;          // DMA instructions per wave, 8 waves
  static constexpr int N4 = BYTES / 1024 / 4;          // 4 waves
  // XOR applied to the chunk index of a row.  Two access patterns must be free of
  // bank conflicts (256 bytes = 16 chunk slots per bank line; with D = 64 two rows
  // share a line): a row-fragment read takes one chunk of 16 consecutive rows, a
  // transposed read takes 4 consecutive chunks (aligned to 4) of 4 consecutive
  // rows (aligned to 4).  So rows that differ in their low bits must land in
  // different aligned groups of 4 chunks, and the 16 rows of a fragment read in 16
  // different slots: the low row bits go to the high chunk bits and vice versa.
  __device__ static __forceinline__ int swz(int row) {
    return CHK == 16 ? (((row & 3) << 2) | ((row >> 2) & 3)) : ((((row >> 1) & 1) << 2) | ((row >> 2) & 3));
  }
  // per-lane byte offset (global side) of DMA instruction `instr` of a tile whose
  // rows are `stride` elements apart
  __device__ static __forceinline__ int voff(int instr, int lane, int64_t stride) {
    const int r = instr * (64 / CHK) + lane / CHK;
    const int c = (lane % CHK) ^ swz(r);
    return (int)(r * stride * 2) + c * 16;
  }
  // row fragment: row `row`, d = 16 s + 8 h ..
  __device__ static __forceinline__ bf16x8 row_frag(const char* tile, int row, int s, int h) {
    return *(const bf16x8*)(tile + row * ROW + (((2 * s + h) ^ swz(row)) * 16));
  }
};

typedef __attribute__((__vector_size__(4 * sizeof(short)))) short shortx4;
typedef __attribute__((address_space(3))) shortx4* lds_shortx4_ptr;

// The LDS transpose read works on groups of 16 lanes: lane 4e+g of a group
// supplies the address of 4 consecutive halfwords, and lane i receives, as
// element e, halfword i%4 of what lane 4e + i/4 addressed.  With lane 4e+g
// pointing at row (k0 + e), columns d0 + 4g .., lane i ends up with column
// d0 + i of rows k0 .. k0+3.
struct TrLane {
  int row_off;   // row this lane addresses, relative to the slab: 4h + e
  int dcol;      // first of its 4 columns, relative to the 32-column tile: 16 (b & 1) + 4 g
  __device__ __forceinline__ TrLane(int lane) {
    const int b = lane >> 4, i = lane & 15;
    row_off = 4 * (b >> 1) + (i >> 2);
    dcol = 16 * (b & 1) + 4 * (i & 3);
  }
};

// Transposed fragment for the 16-row slab starting at row k0 and the 32 columns
// starting at d0: lane (m, h) gets column d0 + m of rows k0 + 4h + {0..3} and
// k0 + 8 + 4h + {0..3} -- the row order in which the accumulator of the score
// tile, used as the other operand, holds a slab.
template <int D>
__device__ __forceinline__ bf16x8 tr_frag(const char* tile, const TrLane& t, int k0, int d0) {
  using T = AttnTile<D>;
  const int col = d0 + t.dcol;
  const int r0 = k0 + t.row_off, r1 = r0 + 8;
  const shortx4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
      (lds_shortx4_ptr)(tile + r0 * T::ROW + (((col >> 3) ^ T::swz(r0)) * 16) + (col & 4) * 2));
  const shortx4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
      (lds_shortx4_ptr)(tile + r1 * T::ROW + (((col >> 3) ^ T::swz(r1)) * 16) + (col & 4) * 2));
  typedef __attribute__((__vector_size__(8 * sizeof(short)))) short shortx8;
  const shortx8 v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  return __builtin_bit_cast(bf16x8, v);
}

// attn_smem_note: the kernels below track the completion of their LDS DMA by hand (wait_vmcnt
// before the barrier that publishes a stage).  Two things would make the compiler drain every
// outstanding DMA instead, serialising the ring: a second LDS variable in the kernel (it then
// puts s_waitcnt vmcnt(0) in front of LDS reads that follow a DMA issue), and __syncthreads(),
// whose fence waits for all memory operations; hence one LDS array per kernel, carved by
// hand, and barrier_lds_only() inside the loops.
// Makes the compiler finish the load of v here (it waits for a value where an instruction first
// uses it).  Left alone it would put the wait for a prologue load at the first use inside the main
// loop, where the same s_waitcnt vmcnt(..) then also waits for the DMA ring on every iteration.
template <class V>
__device__ __forceinline__ void pin_loaded(V& v) {
  asm volatile("" : "+v"(v));
}

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

__device__ __forceinline__ dma_rsrc_t attn_rsrc(const void* p) { return dma_make_rsrc(p, 0x7fffffffu); }

// ----------------------------------------------------------------------------
// Forward
// ----------------------------------------------------------------------------
struct AttnFwdParams {
  const uint16_t* Q;   // element (s, h, d) at s * q_ss + h * q_hs + d
  const uint16_t* K;
  const uint16_t* V;
  uint16_t* O;
  float* lse;          // [Hq][S], natural log
  int64_t q_ss, q_hs, k_ss, k_hs, v_ss, v_hs, o_ss, o_hs;
  const int* gc;
  const int* pc;
  const uint32_t* list;
  const int* cnt;
  int S, Hq, Hkv, nQb, nKb;
  float scale_log2e;
};

// LDS stage of the forward and dQ kernels: K tile, V tile, 64 key codes.
template <int D>
struct AttnKvStage {
  using T = AttnTile<D>;
  static constexpr int V_OFF = T::BYTES;
  static constexpr int CODE_OFF = 2 * T::BYTES;
  static constexpr int STAGE = CODE_OFF + 1024;
  static constexpr int N_PER = 2 * T::N8 + 1;
};

// DMA of key block kb into one stage: this wave's share of the K and V tiles,
// plus the 64 key codes (every wave writes the same 256 bytes).
template <int D>
__device__ __forceinline__ void attn_issue_kv(char* st, int kb, dma_rsrc_t rsrc_k,
                                              dma_rsrc_t rsrc_v,
                                              dma_rsrc_t rsrc_c,
                                              const int* voff_k,
                                              const int* voff_v, int64_t k_ss,
                                              int64_t v_ss, int wave, int lane) {
  using T = AttnTile<D>;
  using G = AttnKvStage<D>;
  const int k0 = kb * ATT_BN;
#pragma unroll
  for (int i = 0; i < T::N8; ++i)
    dma_load16(rsrc_k, voff_k[i], (int)(k0 * k_ss * 2), lds_addr_of(st + (wave * T::N8 + i) * 1024));
#pragma unroll
  for (int i = 0; i < T::N8; ++i)
    dma_load16(rsrc_v, voff_v[i], (int)(k0 * v_ss * 2), lds_addr_of(st + G::V_OFF + (wave * T::N8 + i) * 1024));
  dma_load4(rsrc_c, lane * 4, k0 * 4, lds_addr_of(st + G::CODE_OFF));
}

template <int D>
__global__ __launch_bounds__(512) void attn_fwd_kernel(AttnFwdParams p) {
  using T = AttnTile<D>;
  using G = AttnKvStage<D>;
  // one LDS object for the stages and the tile list (see attn_smem_note)
  __shared__ __attribute__((aligned(1024))) char smem[ATT_STAGES * G::STAGE + ATT_MAX_KB * 4];
  uint32_t* const s_list = (uint32_t*)(smem + ATT_STAGES * G::STAGE);
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int n = lane & 31, h = lane >> 5;
  const TrLane tr(lane);
  const int hq = blockIdx.x % p.Hq;
  const int qb = p.nQb - 1 - (int)(blockIdx.x / p.Hq);  // long rows first
  const int hkv = hq / (p.Hq / p.Hkv);
  const int q = qb * ATT_BM + wave * 32 + n;
  const int cnt = p.cnt[qb];

  for (int i = threadIdx.x; i < cnt; i += 512) s_list[i] = p.list[(int64_t)qb * p.nKb + i];

  // this lane's query as B-operand fragments of S^T = K Q^T
  bf16x8 qf[D / 16];
  {
    const uint16_t* qp = p.Q + (int64_t)q * p.q_ss + (int64_t)hq * p.q_hs + 8 * h;
#pragma unroll
    for (int s = 0; s < D / 16; ++s) qf[s] = *(const bf16x8*)(qp + 16 * s);
  }
  int gi = p.gc[q], pi = p.pc[q];

  const dma_rsrc_t rsrc_k = attn_rsrc(p.K + (int64_t)hkv * p.k_hs);
  const dma_rsrc_t rsrc_v = attn_rsrc(p.V + (int64_t)hkv * p.v_hs);
  const dma_rsrc_t rsrc_c = attn_rsrc(p.gc);
  int voff_k[T::N8], voff_v[T::N8];
#pragma unroll
  for (int i = 0; i < T::N8; ++i) {
    voff_k[i] = T::voff(wave * T::N8 + i, lane, p.k_ss);
    voff_v[i] = T::voff(wave * T::N8 + i, lane, p.v_ss);
  }
  __syncthreads();  // s_list
  auto* list_lds = s_list;
#define ATTN_ISSUE(IT, STG)                                                                          \
  attn_issue_kv<D>(smem + (STG) * G::STAGE, __builtin_amdgcn_readfirstlane(list_lds[IT] & 0x3fff),    \
                   rsrc_k, rsrc_v, rsrc_c, voff_k, voff_v, p.k_ss, p.v_ss, wave, lane)

  floatx16 o[D / 32];
#pragma unroll
  for (int dt = 0; dt < D / 32; ++dt)
#pragma unroll
    for (int j = 0; j < 16; ++j) o[dt][j] = 0.f;
  float m_run = -1e30f, l_run = 0.f;

#pragma unroll
  for (int s = 0; s < D / 16; ++s) pin_loaded(qf[s]);
  pin_loaded(gi);
  pin_loaded(pi);
  if (cnt > 0) ATTN_ISSUE(0, 0);
  if (cnt > 1) ATTN_ISSUE(1, 1);
  int stage = 0;
  for (int it = 0; it < cnt; ++it) {
    if (it + 1 < cnt)
      wait_vmcnt<G::N_PER>();
    else
      wait_vmcnt<0>();
    barrier_lds_only();
    if (it + 2 < cnt) ATTN_ISSUE(it + 2, stage >= 1 ? stage - 1 : ATT_STAGES - 1);
    const int entry = __builtin_amdgcn_readfirstlane(s_list[it]);
    const int kb = entry & 0x3fff;
    const bool active = (entry >> (16 + wave)) & 1;        // this wave's 32 queries see part of the tile
    const bool partial = !((entry >> (24 + wave)) & 1);     // ... but not all of it
    const char* st = smem + stage * G::STAGE;
    stage = stage + 1 == ATT_STAGES ? 0 : stage + 1;
    if (!active) continue;  // nothing of this tile is visible to this wave's queries

    // S^T tiles: keys 0..31 and 32..63 of the block x this wave's 32 queries
    floatx16 sc[2];
#pragma unroll
    for (int j = 0; j < 16; ++j) sc[0][j] = sc[1][j] = 0.f;
    {
      // K fragments three steps ahead of the MFMAs that use them (LDS latency)
      constexpr int NS = D / 16, PF = 3;
      bf16x8 kf[NS][2];
#pragma unroll
      for (int s = 0; s < PF; ++s) {
        kf[s][0] = T::row_frag(st, n, s, h);
        kf[s][1] = T::row_frag(st, 32 + n, s, h);
      }
      __builtin_amdgcn_sched_group_barrier(0x100, 2 * PF, 0);
#pragma unroll
      for (int s = 0; s < NS; ++s) {
        if (s + PF < NS) {
          kf[s + PF][0] = T::row_frag(st, n, s + PF, h);
          kf[s + PF][1] = T::row_frag(st, 32 + n, s + PF, h);
        }
        sc[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[s][0], qf[s], sc[0], 0, 0, 0);
        sc[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[s][1], qf[s], sc[1], 0, 0, 0);
        if (s + PF < NS) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
      }
    }

    // mask, running max (of the raw scores: the scale is positive and rides in the exponent's
    // multiply-add below)
    float mloc = -INFINITY;
    if (partial) {
      const int* codes = (const int*)(st + G::CODE_OFF);
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) {
          const int kk = 32 * kt + 8 * g4 + 4 * h;
          const int4 kc = *(const int4*)(codes + kk);
          const int key = kb * ATT_BN + kk;
          const int kcv[4] = {kc.x, kc.y, kc.z, kc.w};
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (!attn_visible(q, key + e, gi, pi, kcv[e])) sc[kt][4 * g4 + e] = -INFINITY;
        }
    }
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int j = 0; j < 16; ++j) mloc = fmaxf(mloc, sc[kt][j]);
    mloc = fmaxf(mloc, __shfl_xor(mloc, 32, 64)) * p.scale_log2e;
    // The reference of the exponentials follows the running maximum lazily: it moves only when
    // some query of the wave has a score more than ATT_LAZY (in units of log2) above it, so the
    // 64 output accumulators are rescaled on few tiles instead of on most early ones.  Until
    // then exponentials are at most 2^ATT_LAZY, which fp32 sums and bf16 operands hold without
    // loss; the final division by the sum is the same.
    const bool move = __any(mloc > m_run + ATT_LAZY);
    float lsum = 0.f;
    bf16x8 pf[4];
    if (move) {
      const float m_new = fmaxf(m_run, mloc);
      const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
      m_run = m_new;
      l_run *= alpha;
#pragma unroll
      for (int dt = 0; dt < D / 32; ++dt)
#pragma unroll
        for (int j = 0; j < 16; ++j) o[dt][j] *= alpha;
    }
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        const float e = __builtin_amdgcn_exp2f(__builtin_fmaf(sc[kt][j], p.scale_log2e, -m_run));
        lsum += e;
        pf[2 * kt + j / 8][j % 8] = (__bf16)e;
      }
    l_run += lsum;

    // O^T += V^T P^T, V^T fragments by transposing reads of the V tile
    const char* vt = st + G::V_OFF;
#pragma unroll
    for (int s2 = 0; s2 < 4; ++s2) {
#pragma unroll
      for (int dt = 0; dt < D / 32; ++dt)
        o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tr_frag<D>(vt, tr, 16 * s2, 32 * dt), pf[s2], o[dt],
                                                        0, 0, 0);
    }
  }
#undef ATTN_ISSUE

  const float l_tot = l_run + __shfl_xor(l_run, 32, 64);
  const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
  uint16_t* op = p.O + (int64_t)q * p.o_ss + (int64_t)hq * p.o_hs + 4 * h;
#pragma unroll
  for (int dt = 0; dt < D / 32; ++dt)
#pragma unroll
    for (int g4 = 0; g4 < 4; ++g4) {
      bf16x4 v;
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = (__bf16)(o[dt][4 * g4 + e] * inv);
      *(bf16x4*)(op + 32 * dt + 8 * g4) = v;
    }
  if (h == 0) p.lse[(int64_t)hq * p.S + q] = (m_run + __builtin_amdgcn_logf(l_tot)) * LN2;
}

// ----------------------------------------------------------------------------
// Backward
//   P = exp(scale * S + bias - lse),  dV = P^T dO,  dP = dO V^T,
//   dS = P o (dP - delta),  delta_i = sum_d dO[i,d] O[i,d],
//   dQ = scale * dS K,  dK = scale * dS^T Q.
// Two kernels, both free of atomics (bit-reproducible): one owns a block of
// keys and accumulates dK, dV over the query tiles that see it, the other owns
// a block of queries and accumulates dQ over its visible key tiles.  Each
// recomputes P from lse.
// ----------------------------------------------------------------------------
struct AttnBwdParams {
  const uint16_t *Q, *K, *V, *dO;
  const float* lse2;                // [Hq][S]  lse * log2(e)
  const float* delta;               // [Hq][S]
  uint16_t *dQ, *dK, *dV;
  float *pK, *pV;                   // [Hq/Hkv][S][Hkv][D] per-head partial sums (grouped-query heads only)
  int64_t q_ss, q_hs, k_ss, k_hs, v_ss, v_hs, do_ss, do_hs, dq_ss, dq_hs, dk_ss, dk_hs, dv_ss, dv_hs;
  const int* gc;
  const int* pc;
  const uint32_t* list;    // per query block of 256: key tiles of 64
  const int* cnt;
  const uint32_t* listT;   // per key block of 128: query tiles of 64
  const int* cntT;
  int S, Hq, Hkv, nQb, nKb, nQb2, nKb2;
  int light_max;           // see ATT_LIGHT_MAX; 0 when there are too few key blocks to fill the GPU that way
  float scale, scale_log2e;
};

// delta[h][s] = sum_d dO[s,h,d] * O[s,h,d] and lse2 = lse * log2(e); 16 lanes per (s, h).
__global__ __launch_bounds__(256) void attn_delta_kernel(const uint16_t* __restrict__ O, int64_t o_ss,
                                                         int64_t o_hs,
                                                         const uint16_t* __restrict__ dO,
                                                         int64_t do_ss, int64_t do_hs,
                                                         const float* __restrict__ lse, int S, int H,
                                                         int D, float* __restrict__ delta,
                                                         float* __restrict__ lse2) {
  const int64_t row = (int64_t)blockIdx.x * 16 + (threadIdx.x >> 4);
  const int sub = threadIdx.x & 15;
  if (row >= (int64_t)S * H) return;
  const int s = (int)(row / H), hh = (int)(row - (int64_t)s * H);
  const uint16_t* op = O + (int64_t)s * o_ss + (int64_t)hh * o_hs;
  const uint16_t* gp = dO + (int64_t)s * do_ss + (int64_t)hh * do_hs;
  float acc = 0.f;
  for (int d = sub * 8; d < D; d += 128) {
    const bf16x8 a = *(const bf16x8*)(op + d);
    const bf16x8 b = *(const bf16x8*)(gp + d);
#pragma unroll
    for (int e = 0; e < 8; ++e) acc += (float)a[e] * (float)b[e];
  }
#pragma unroll
  for (int o = 8; o > 0; o >>= 1) acc += __shfl_xor(acc, o, 64);
  if (sub == 0) {
    delta[(int64_t)hh * S + s] = acc;
    lse2[(int64_t)hh * S + s] = lse[(int64_t)hh * S + s] * LOG2E;
  }
}

// ---- dQ: 256 queries x one head per work-group, lane = query ----------------
template <int D>
__global__ __launch_bounds__(512) void attn_bwd_dq_kernel(AttnBwdParams p) {
  using T = AttnTile<D>;
  using G = AttnKvStage<D>;
  // one LDS object for the stages and the tile list (see attn_smem_note)
  __shared__ __attribute__((aligned(1024))) char smem[ATT_STAGES * G::STAGE + ATT_MAX_KB * 4];
  uint32_t* const s_list = (uint32_t*)(smem + ATT_STAGES * G::STAGE);
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int n = lane & 31, h = lane >> 5;
  const TrLane tr(lane);
  const int hq = blockIdx.x % p.Hq;
  const int qb = p.nQb - 1 - (int)(blockIdx.x / p.Hq);
  const int hkv = hq / (p.Hq / p.Hkv);
  const int q = qb * ATT_BM + wave * 32 + n;
  const int cnt = p.cnt[qb];
  for (int i = threadIdx.x; i < cnt; i += 512) s_list[i] = p.list[(int64_t)qb * p.nKb + i];

  bf16x8 qf[D / 16], dof[D / 16];
  {
    const uint16_t* qp = p.Q + (int64_t)q * p.q_ss + (int64_t)hq * p.q_hs + 8 * h;
    const uint16_t* gp = p.dO + (int64_t)q * p.do_ss + (int64_t)hq * p.do_hs + 8 * h;
#pragma unroll
    for (int s = 0; s < D / 16; ++s) {
      qf[s] = *(const bf16x8*)(qp + 16 * s);
      dof[s] = *(const bf16x8*)(gp + 16 * s);
    }
  }
  int gi = p.gc[q], pi = p.pc[q];
  float nlse2 = -p.lse2[(int64_t)hq * p.S + q];
  float delta = p.delta[(int64_t)hq * p.S + q];

  const dma_rsrc_t rsrc_k = attn_rsrc(p.K + (int64_t)hkv * p.k_hs);
  const dma_rsrc_t rsrc_v = attn_rsrc(p.V + (int64_t)hkv * p.v_hs);
  const dma_rsrc_t rsrc_c = attn_rsrc(p.gc);
  int voff_k[T::N8], voff_v[T::N8];
#pragma unroll
  for (int i = 0; i < T::N8; ++i) {
    voff_k[i] = T::voff(wave * T::N8 + i, lane, p.k_ss);
    voff_v[i] = T::voff(wave * T::N8 + i, lane, p.v_ss);
  }
  __syncthreads();
  auto* list_lds = s_list;
#define ATTN_ISSUE(IT, STG)                                                                          \
  attn_issue_kv<D>(smem + (STG) * G::STAGE, __builtin_amdgcn_readfirstlane(list_lds[IT] & 0x3fff),    \
                   rsrc_k, rsrc_v, rsrc_c, voff_k, voff_v, p.k_ss, p.v_ss, wave, lane)

  floatx16 dq[D / 32];
#pragma unroll
  for (int dt = 0; dt < D / 32; ++dt)
#pragma unroll
    for (int j = 0; j < 16; ++j) dq[dt][j] = 0.f;

#pragma unroll
  for (int s = 0; s < D / 16; ++s) {
    pin_loaded(qf[s]);
    pin_loaded(dof[s]);
  }
  pin_loaded(gi);
  pin_loaded(pi);
  pin_loaded(nlse2);
  pin_loaded(delta);
  if (cnt > 0) ATTN_ISSUE(0, 0);
  if (cnt > 1) ATTN_ISSUE(1, 1);
  int stage = 0;
  for (int it = 0; it < cnt; ++it) {
    if (it + 1 < cnt)
      wait_vmcnt<G::N_PER>();
    else
      wait_vmcnt<0>();
    barrier_lds_only();
    if (it + 2 < cnt) ATTN_ISSUE(it + 2, stage >= 1 ? stage - 1 : ATT_STAGES - 1);
    const int entry = __builtin_amdgcn_readfirstlane(s_list[it]);
    const int kb = entry & 0x3fff;
    const bool active = (entry >> (16 + wave)) & 1;        // this wave's 32 queries see part of the tile
    const bool partial = !((entry >> (24 + wave)) & 1);     // ... but not all of it
    const char* st = smem + stage * G::STAGE;
    const int* codes = (const int*)(st + G::CODE_OFF);
    stage = stage + 1 == ATT_STAGES ? 0 : stage + 1;
    if (!active) continue;

    bf16x8 dsf[4];
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) {
      floatx16 sc, dp;
#pragma unroll
      for (int j = 0; j < 16; ++j) sc[j] = dp[j] = 0.f;
#pragma unroll
      for (int s = 0; s < D / 16; ++s) {
        sc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(T::row_frag(st, 32 * kt + n, s, h), qf[s], sc, 0, 0, 0);
        dp = __builtin_amdgcn_mfma_f32_32x32x16_bf16(T::row_frag(st + G::V_OFF, 32 * kt + n, s, h), dof[s],
                                                     dp, 0, 0, 0);
      }
#pragma unroll
      for (int g4 = 0; g4 < 4; ++g4) {
        const int kk = 32 * kt + 8 * g4 + 4 * h;
        int kcv[4] = {0, 0, 0, 0};
        if (partial) {
          const int4 kc = *(const int4*)(codes + kk);
          kcv[0] = kc.x; kcv[1] = kc.y; kcv[2] = kc.z; kcv[3] = kc.w;
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int j = 4 * g4 + e;
          float x = __builtin_fmaf(sc[j], p.scale_log2e, nlse2);
          if (partial && !attn_visible(q, kb * ATT_BN + kk + e, gi, pi, kcv[e])) x = -INFINITY;
          const float pr = __builtin_amdgcn_exp2f(x);
          dsf[2 * kt + j / 8][j % 8] = (__bf16)(pr * (dp[j] - delta));
        }
      }
    }
    // dQ^T += K^T dS^T, K^T fragments by transposing reads of the K tile
#pragma unroll
    for (int s2 = 0; s2 < 4; ++s2) {
#pragma unroll
      for (int dt = 0; dt < D / 32; ++dt)
        dq[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tr_frag<D>(st, tr, 16 * s2, 32 * dt), dsf[s2], dq[dt],
                                                         0, 0, 0);
    }
  }
#undef ATTN_ISSUE
  uint16_t* op = p.dQ + (int64_t)q * p.dq_ss + (int64_t)hq * p.dq_hs + 4 * h;
#pragma unroll
  for (int dt = 0; dt < D / 32; ++dt)
#pragma unroll
    for (int g4 = 0; g4 < 4; ++g4) {
      bf16x4 v;
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = (__bf16)(dq[dt][4 * g4 + e] * p.scale);
      *(bf16x4*)(op + 32 * dt + 8 * g4) = v;
    }
}

// ---- dK, dV: 128 keys x one query head per work-group, lane = key ------------
// 8 wavefronts = 4 key groups of 32 x 2 halves of each 64-query tile, so every
// SIMD holds two waves and the exp2 / convert work of one overlaps the MFMAs of
// the other.  The two waves of a key group keep separate accumulators, added
// through LDS at the end.  The K and V rows of the block stay in LDS for the
// whole kernel (their fragments are re-read per tile: keeping them in
// registers would push a wave past 256 registers).
// With grouped-query heads the work-groups of the heads that share a key/value
// head write fp32 partial sums, which attn_kv_reduce_kernel adds in a fixed order.
// LDS stage: Q tile, dO tile (64 queries), and lse2 / delta / group / parent codes
// of those queries.
template <int D>
struct AttnQStage {
  using T = AttnTile<D>;
  static constexpr int DO_OFF = T::BYTES;
  static constexpr int ROW_OFF = 2 * T::BYTES;
  static constexpr int STAGE = ROW_OFF + 1024;
  static constexpr int NSTAGE = 2;
  static constexpr int KV_OFF = NSTAGE * STAGE;          // K block (2 tiles), then V block
  static constexpr int LDS = KV_OFF + 4 * T::BYTES;
};

// DMA of one query tile into a stage: this wave's share of the Q and dO tiles and
// one of the four per-query arrays (wave & 3 = 0: lse2, 1: delta, 2: group codes,
// 3: parent codes; the upper four waves write the same bytes again).
template <int D>
__device__ __forceinline__ void attn_issue_q(char* st, int hq, int q0, dma_rsrc_t rsrc_q,
                                             dma_rsrc_t rsrc_do,
                                             dma_rsrc_t rsrc_row, const int* voff_q,
                                             const int* voff_do, const AttnBwdParams& p, int wave,
                                             int lane) {
  using T = AttnTile<D>;
  using G = AttnQStage<D>;
  const int so_q = (int)((q0 * p.q_ss + hq * p.q_hs) * 2);
  const int so_do = (int)((q0 * p.do_ss + hq * p.do_hs) * 2);
#pragma unroll
  for (int i = 0; i < T::N8; ++i) {
    dma_load16(rsrc_q, voff_q[i], so_q, lds_addr_of(st + (wave * T::N8 + i) * 1024));
    dma_load16(rsrc_do, voff_do[i], so_do, lds_addr_of(st + G::DO_OFF + (wave * T::N8 + i) * 1024));
  }
  const int arr = wave & 3;
  dma_load4(rsrc_row, lane * 4, (int)(((arr < 2 ? (int64_t)hq * p.S : 0) + q0) * 4), lds_addr_of(st + G::ROW_OFF + arr * 256));
}

// The block's K and V rows (128 each = two 64-row tiles per operand).
template <int D>
__device__ __forceinline__ void attn_issue_kv_block(char* dst, int key0, dma_rsrc_t rsrc_k,
                                                    dma_rsrc_t rsrc_v, const int* voff_k,
                                                    const int* voff_v, int64_t k_ss, int64_t v_ss,
                                                    int wave) {
  using T = AttnTile<D>;
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int i = 0; i < T::N8; ++i) {
      dma_load16(rsrc_k, voff_k[i], (int)((key0 + 64 * t) * k_ss * 2), lds_addr_of(dst + t * T::BYTES + (wave * T::N8 + i) * 1024));
      dma_load16(rsrc_v, voff_v[i], (int)((key0 + 64 * t) * v_ss * 2), lds_addr_of(dst + (2 + t) * T::BYTES + (wave * T::N8 + i) * 1024));
    }
}

template <int D>
__global__ __launch_bounds__(512) void attn_bwd_kv_kernel(AttnBwdParams p) {
  using T = AttnTile<D>;
  using G = AttnQStage<D>;
  // one LDS object for the stages and the tile list (see attn_smem_note)
  __shared__ __attribute__((aligned(1024))) char smem[G::LDS + ATT_MAX_KB * 4];
  uint32_t* const s_list = (uint32_t*)(smem + G::LDS);
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int n = lane & 31, h = lane >> 5;
  const int kg = wave & 3, qh = wave >> 2;
  const TrLane tr(lane);
  const int hq = blockIdx.x % p.Hq;
  const int kb = (int)(blockIdx.x / p.Hq);  // early key blocks are seen by the most queries
  const int rep = p.Hq / p.Hkv;
  const int hkv = hq / rep;
  const int key = kb * ATT_BK2 + kg * 32 + n;
  const int cnt = p.cntT[kb];
  const bool light = rep > 1 && cnt * rep <= p.light_max;
  if (light && hq != hkv * rep) return;  // the group's first head does all of them
  const int nheads = light ? rep : 1;
  for (int i = threadIdx.x; i < cnt; i += 512) s_list[i] = p.listT[(int64_t)kb * p.nQb2 + i];
  int gk = p.gc[key];

  const dma_rsrc_t rsrc_q = attn_rsrc(p.Q);
  const dma_rsrc_t rsrc_do = attn_rsrc(p.dO);
  const int arr = wave & 3;
  const void* row_src = arr == 0 ? (const void*)p.lse2 : arr == 1 ? (const void*)p.delta
                        : arr == 2 ? (const void*)p.gc : (const void*)p.pc;
  const dma_rsrc_t rsrc_row = attn_rsrc(row_src);
  int voff_q[T::N8], voff_do[T::N8];
  {
    int voff_k[T::N8], voff_v[T::N8];
#pragma unroll
    for (int i = 0; i < T::N8; ++i) {
      voff_q[i] = T::voff(wave * T::N8 + i, lane, p.q_ss);
      voff_do[i] = T::voff(wave * T::N8 + i, lane, p.do_ss);
      voff_k[i] = T::voff(wave * T::N8 + i, lane, p.k_ss);
      voff_v[i] = T::voff(wave * T::N8 + i, lane, p.v_ss);
    }
    attn_issue_kv_block<D>(smem + G::KV_OFF, kb * ATT_BK2, attn_rsrc(p.K + (int64_t)hkv * p.k_hs),
                           attn_rsrc(p.V + (int64_t)hkv * p.v_hs), voff_k, voff_v, p.k_ss, p.v_ss, wave);
  }
  __syncthreads();  // s_list
  auto* list_lds = s_list;
  // step IT of the flattened (head, visible query tile) sequence
#define ATTN_ISSUE(IT, STG)                                                                          \
  do {                                                                                               \
    const int hi_ = (IT) / cnt, ti_ = (IT) - hi_ * cnt;                                               \
    attn_issue_q<D>(smem + (STG) * G::STAGE, hq + hi_,                                                \
                    __builtin_amdgcn_readfirstlane(list_lds[ti_] & 0x3fff) * ATT_BQ2, rsrc_q, rsrc_do, \
                    rsrc_row, voff_q, voff_do, p, wave, lane);                                        \
  } while (0)

  floatx16 dk[D / 32], dv[D / 32];
#pragma unroll
  for (int dt = 0; dt < D / 32; ++dt)
#pragma unroll
    for (int j = 0; j < 16; ++j) dk[dt][j] = dv[dt][j] = 0.f;

  // this wave's keys inside the resident K / V blocks
  const char* kblk = smem + G::KV_OFF + (kg >> 1) * T::BYTES;
  const char* vblk = kblk + 2 * T::BYTES;
  const int krow = 32 * (kg & 1) + n;

  const int total = cnt * nheads;
  pin_loaded(gk);
  if (total > 0) ATTN_ISSUE(0, 0);
  int ti = 0;
  for (int it = 0; it < total; ++it) {
    wait_vmcnt<0>();
    barrier_lds_only();
    if (it + 1 < total) ATTN_ISSUE(it + 1, (it + 1) & 1);
    const int entry = __builtin_amdgcn_readfirstlane(s_list[ti]);
    ti = ti + 1 == cnt ? 0 : ti + 1;
    const int q0 = (entry & 0x3fff) * ATT_BQ2;
    const bool active = (entry >> (16 + wave)) & 1;        // this wave's keys x query half
    const bool partial = !((entry >> (24 + wave)) & 1);
    const char* st = smem + (it & 1) * G::STAGE;
    const char* dot = st + G::DO_OFF;
    const float* r_lse2 = (const float*)(st + G::ROW_OFF);
    const float* r_delta = r_lse2 + 64;
    const int* r_gc = (const int*)(r_lse2 + 128);
    const int* r_pc = r_gc + 64;
    if (!active) continue;

    floatx16 sc, dp;
#pragma unroll
    for (int j = 0; j < 16; ++j) sc[j] = dp[j] = 0.f;
#pragma unroll
    for (int s = 0; s < D / 16; ++s) {
      sc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(T::row_frag(st, 32 * qh + n, s, h),
                                                   T::row_frag(kblk, krow, s, h), sc, 0, 0, 0);
      dp = __builtin_amdgcn_mfma_f32_32x32x16_bf16(T::row_frag(dot, 32 * qh + n, s, h),
                                                   T::row_frag(vblk, krow, s, h), dp, 0, 0, 0);
    }
    bf16x8 pf[2], dsf[2];
#pragma unroll
    for (int g4 = 0; g4 < 4; ++g4) {
      const int qi = 32 * qh + 8 * g4 + 4 * h;
      const floatx4 l4 = *(const floatx4*)(r_lse2 + qi);
      const floatx4 d4 = *(const floatx4*)(r_delta + qi);
      int gq[4] = {0, 0, 0, 0}, pq[4] = {0, 0, 0, 0};
      if (partial) {
        const int4 a4 = *(const int4*)(r_gc + qi);
        const int4 b4 = *(const int4*)(r_pc + qi);
        gq[0] = a4.x; gq[1] = a4.y; gq[2] = a4.z; gq[3] = a4.w;
        pq[0] = b4.x; pq[1] = b4.y; pq[2] = b4.z; pq[3] = b4.w;
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int j = 4 * g4 + e;
        float x = __builtin_fmaf(sc[j], p.scale_log2e, -l4[e]);
        if (partial && !attn_visible(q0 + qi + e, key, gq[e], pq[e], gk)) x = -INFINITY;
        const float pr = __builtin_amdgcn_exp2f(x);
        pf[j / 8][j % 8] = (__bf16)pr;
        dsf[j / 8][j % 8] = (__bf16)(pr * (dp[j] - d4[e]));
      }
    }
    // dV^T += dO^T P, dK^T += Q^T dS: transposing reads of the dO and Q tiles
#pragma unroll
    for (int u = 0; u < 2; ++u) {
#pragma unroll
      for (int dt = 0; dt < D / 32; ++dt) {
        dv[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tr_frag<D>(dot, tr, 32 * qh + 16 * u, 32 * dt), pf[u],
                                                         dv[dt], 0, 0, 0);
        dk[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tr_frag<D>(st, tr, 32 * qh + 16 * u, 32 * dt), dsf[u],
                                                         dk[dt], 0, 0, 0);
      }
    }
  }
#undef ATTN_ISSUE

  // add the accumulators of the two query halves: the upper waves park theirs in
  // LDS ([key group][register][lane], conflict-free), the lower waves add and store
  float* red = (float*)smem;
#pragma unroll
  for (int pass = 0; pass < 2; ++pass) {
    __syncthreads();
    if (qh == 1) {
#pragma unroll
      for (int dt = 0; dt < D / 32; ++dt)
#pragma unroll
        for (int j = 0; j < 16; ++j)
          red[((kg * (D / 2) + dt * 16 + j) << 6) + lane] = pass == 0 ? dk[dt][j] : dv[dt][j];
    }
    __syncthreads();
    if (qh == 0) {
#pragma unroll
      for (int dt = 0; dt < D / 32; ++dt)
#pragma unroll
        for (int j = 0; j < 16; ++j) {
          const float v = red[((kg * (D / 2) + dt * 16 + j) << 6) + lane];
          if (pass == 0) dk[dt][j] += v; else dv[dt][j] += v;
        }
    }
  }
  if (qh == 1) return;

  if (rep > 1 && !light) {
    const int64_t o = ((((int64_t)(hq - hkv * rep) * p.S + key) * p.Hkv + hkv) * D) + 4 * h;
#pragma unroll
    for (int dt = 0; dt < D / 32; ++dt)
#pragma unroll
      for (int g4 = 0; g4 < 4; ++g4) {
        floatx4 a, b;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          a[e] = dk[dt][4 * g4 + e];
          b[e] = dv[dt][4 * g4 + e];
        }
        *(floatx4*)(p.pK + o + 32 * dt + 8 * g4) = a;
        *(floatx4*)(p.pV + o + 32 * dt + 8 * g4) = b;
      }
    return;
  }
  uint16_t* kp = p.dK + (int64_t)key * p.dk_ss + (int64_t)hkv * p.dk_hs + 4 * h;
  uint16_t* vp = p.dV + (int64_t)key * p.dv_ss + (int64_t)hkv * p.dv_hs + 4 * h;
#pragma unroll
  for (int dt = 0; dt < D / 32; ++dt)
#pragma unroll
    for (int g4 = 0; g4 < 4; ++g4) {
      bf16x4 a, b;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        a[e] = (__bf16)(dk[dt][4 * g4 + e] * p.scale);
        b[e] = (__bf16)dv[dt][4 * g4 + e];
      }
      *(bf16x4*)(kp + 32 * dt + 8 * g4) = a;
      *(bf16x4*)(vp + 32 * dt + 8 * g4) = b;
    }
}

// dK = scale * sum_r pK[r], dV = sum_r pV[r] over the query heads r of a group, in
// index order; 4 elements per thread.
__global__ __launch_bounds__(256) void attn_kv_reduce_kernel(const float* __restrict__ pK,
                                                             const float* __restrict__ pV,
                                                             const int* __restrict__ cntT,
                                                             int light_max, int rep,
                                                             int64_t S, int Hkv, int D, float scale,
                                                             uint16_t* __restrict__ dK, int64_t dk_ss,
                                                             int64_t dk_hs, uint16_t* __restrict__ dV,
                                                             int64_t dv_ss, int64_t dv_hs) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int d4 = D / 4;
  const int64_t n = S * Hkv * d4;
  if (i >= n) return;
  const int c = (int)(i % d4);
  const int hh = (int)((i / d4) % Hkv);
  const int64_t s = i / ((int64_t)d4 * Hkv);
  if (cntT[s / ATT_BK2] * rep <= light_max) return;  // written directly by the dK/dV kernel
  floatx4 a = {0.f, 0.f, 0.f, 0.f}, b = {0.f, 0.f, 0.f, 0.f};
  for (int r = 0; r < rep; ++r) {
    a += ((const floatx4*)pK)[(int64_t)r * n + i];
    b += ((const floatx4*)pV)[(int64_t)r * n + i];
  }
  bf16x4 oa, ob;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    oa[e] = (__bf16)(a[e] * scale);
    ob[e] = (__bf16)b[e];
  }
  *(bf16x4*)(dK + s * dk_ss + (int64_t)hh * dk_hs + 4 * c) = oa;
  *(bf16x4*)(dV + s * dv_ss + (int64_t)hh * dv_hs + 4 * c) = ob;
}

}  // namespace artk

// Threshold override of artk_attn_bwd_tuning for calls made on this thread (-1: automatic).
static thread_local int g_light_max_override = -1;

using namespace artk;

extern "C" {

size_t artk_attn_plan_bytes(int64_t S) {
  AttnPlan pl;
  return attn_plan_layout(nullptr, 0, S, pl) + 256;
}

int32_t artk_attn_plan(const int64_t* group_ids, const int64_t* parent_ids, int64_t S, void* plan,
                       size_t plan_bytes, artk_stream_t stream) {
  ARTK_CHECK_ARG(group_ids && parent_ids && plan, "null pointer argument");
  ARTK_CHECK_ARG(S > 0, "S must be positive");
  if (S % ATT_BM != 0 || S / ATT_BN > ATT_MAX_KB) {
    set_error("row length %lld must be a multiple of %d and at most %d", (long long)S, ATT_BM,
              ATT_MAX_KB * ATT_BN);
    return ARTK_ERR_UNSUPPORTED_SHAPE;
  }
  AttnPlan pl;
  if (attn_plan_layout(plan, plan_bytes, S, pl) == (size_t)-1) {
    set_error("plan buffer too small: need %zu bytes, got %zu", artk_attn_plan_bytes(S), plan_bytes);
    return ARTK_ERR_WORKSPACE_TOO_SMALL;
  }
  hipStream_t st = (hipStream_t)stream;
  attn_codes_kernel<<<(unsigned)(S / 256), 256, 0, st>>>(group_ids, parent_ids, (int)S, pl.gc, pl.pc);
  ARTK_CHECK_LAUNCH();
  attn_classify_kernel<0><<<dim3((unsigned)((pl.nKb + 3) / 4), (unsigned)pl.nQb), 256, 0, st>>>(
      pl.gc, pl.pc, pl.nKb, pl.info);
  ARTK_CHECK_LAUNCH();
  attn_compact_kernel<<<(unsigned)pl.nQb, 256, 0, st>>>(pl.info, pl.nKb, pl.list, pl.cnt);
  ARTK_CHECK_LAUNCH();
  attn_classify_kernel<1><<<dim3((unsigned)((pl.nQb2 + 3) / 4), (unsigned)pl.nKb2), 256, 0, st>>>(
      pl.gc, pl.pc, pl.nQb2, pl.info2);
  ARTK_CHECK_LAUNCH();
  attn_compact_kernel<<<(unsigned)pl.nKb2, 256, 0, st>>>(pl.info2, pl.nQb2, pl.list2, pl.cnt2);
  ARTK_CHECK_LAUNCH();
  return ARTK_OK;
}

static int32_t attn_check(int64_t S, int32_t Hq, int32_t Hkv, int32_t D, const int64_t* strides,
                          int nstrides) {
  ARTK_CHECK_ARG(S > 0 && Hq > 0 && Hkv > 0, "S, Hq, Hkv must be positive");
  if (S % ATT_BM != 0 || S / ATT_BN > ATT_MAX_KB) {
    set_error("row length %lld must be a multiple of %d and at most %d", (long long)S, ATT_BM,
              ATT_MAX_KB * ATT_BN);
    return ARTK_ERR_UNSUPPORTED_SHAPE;
  }
  if (D != 64 && D != 128) {
    set_error("head dimension %d is not supported (64 or 128)", D);
    return ARTK_ERR_UNSUPPORTED_SHAPE;
  }
  if (Hq % Hkv != 0) {
    set_error("query heads (%d) must be a multiple of key/value heads (%d)", Hq, Hkv);
    return ARTK_ERR_UNSUPPORTED_SHAPE;
  }
  for (int i = 0; i < nstrides; ++i) {
    ARTK_CHECK_ARG(strides[i] > 0 && strides[i] % 8 == 0, "strides must be positive multiples of 8 elements");
    ARTK_CHECK_ARG(i % 2 != 0 || S * strides[i] * 2 < (1ll << 31), "operand spans 2 GiB or more");
  }
  return ARTK_OK;
}

size_t artk_attn_fwd_workspace_bytes(int64_t S, int32_t Hkv, int32_t D) {
  (void)S; (void)Hkv; (void)D;
  return 256;  // the forward needs no scratch; kept so that every op has the same calling pattern
}

int32_t artk_attn_fwd(const void* q, const void* k, const void* v, const void* plan, int64_t S,
                      int32_t Hq, int32_t Hkv, int32_t D, int64_t q_stride_s, int64_t q_stride_h,
                      int64_t k_stride_s, int64_t k_stride_h, int64_t v_stride_s, int64_t v_stride_h,
                      int64_t o_stride_s, int64_t o_stride_h, float scale, void* out, float* lse,
                      void* workspace, size_t workspace_bytes, artk_stream_t stream) {
  ARTK_CHECK_ARG(q && k && v && plan && out && lse, "null pointer argument");
  ARTK_CHECK_ARG(aligned16(q) && aligned16(k) && aligned16(v) && aligned16(out),
                 "q, k, v, out must be 16-byte aligned");
  const int64_t strides[8] = {q_stride_s, q_stride_h, k_stride_s, k_stride_h,
                              v_stride_s, v_stride_h, o_stride_s, o_stride_h};
  int32_t rc = attn_check(S, Hq, Hkv, D, strides, 8);
  if (rc) return rc;
  ARTK_CHECK_ARG(scale > 0.f && scale < INFINITY, "scale must be positive and finite");
  (void)workspace; (void)workspace_bytes;
  AttnPlan pl;
  attn_plan_layout(const_cast<void*>(plan), (size_t)1 << 40, S, pl);
  hipStream_t st = (hipStream_t)stream;
  AttnFwdParams p;
  p.Q = (const uint16_t*)q;
  p.K = (const uint16_t*)k;
  p.V = (const uint16_t*)v;
  p.O = (uint16_t*)out;
  p.lse = lse;
  p.q_ss = q_stride_s;
  p.q_hs = q_stride_h;
  p.k_ss = k_stride_s;
  p.k_hs = k_stride_h;
  p.v_ss = v_stride_s;
  p.v_hs = v_stride_h;
  p.o_ss = o_stride_s;
  p.o_hs = o_stride_h;
  p.gc = pl.gc;
  p.pc = pl.pc;
  p.list = pl.list;
  p.cnt = pl.cnt;
  p.S = (int)S;
  p.Hq = Hq;
  p.Hkv = Hkv;
  p.nQb = pl.nQb;
  p.nKb = pl.nKb;
  p.scale_log2e = scale * LOG2E;
  const unsigned grid = (unsigned)(pl.nQb * Hq);
  prof_begin(PROF_ATTN_FWD, st);
  if (D == 128)
    attn_fwd_kernel<128><<<grid, 512, 0, st>>>(p);
  else
    attn_fwd_kernel<64><<<grid, 512, 0, st>>>(p);
  prof_end(PROF_ATTN_FWD, st);
  ARTK_CHECK_LAUNCH();
  return ARTK_OK;
}

size_t artk_attn_bwd_workspace_bytes(int64_t S, int32_t Hq, int32_t Hkv, int32_t D) {
  Workspace ws(nullptr, 0);
  ws.take<float>((size_t)S * Hq);
  ws.take<float>((size_t)S * Hq);
  if (Hq != Hkv) {
    ws.take<float>((size_t)S * Hq * D);
    ws.take<float>((size_t)S * Hq * D);
  }
  return ws.used + 256;
}

int32_t artk_attn_bwd(const void* q, const void* k, const void* v, const void* out, const float* lse,
                      const void* d_out, const void* plan, int64_t S, int32_t Hq, int32_t Hkv,
                      int32_t D, const int64_t* strides, float scale, void* dq, void* dk, void* dv,
                      void* workspace, size_t workspace_bytes, artk_stream_t stream) {
  ARTK_CHECK_ARG(q && k && v && out && lse && d_out && plan && strides && dq && dk && dv,
                 "null pointer argument");
  ARTK_CHECK_ARG(aligned16(q) && aligned16(k) && aligned16(v) && aligned16(out) && aligned16(d_out) &&
                     aligned16(dq) && aligned16(dk) && aligned16(dv),
                 "tensors must be 16-byte aligned");
  int32_t rc = attn_check(S, Hq, Hkv, D, strides, 16);
  if (rc) return rc;
  // the dK/dV kernel addresses q and d_out by head through 31-bit offsets
  ARTK_CHECK_ARG((S * strides[0] + Hq * strides[1]) * 2 < (1ll << 31) &&
                     (S * strides[8] + Hq * strides[9]) * 2 < (1ll << 31) && (int64_t)S * Hq * 4 < (1ll << 31),
                 "q / d_out span 2 GiB or more");
  Workspace ws(workspace, workspace_bytes);
  float* delta = ws.take<float>((size_t)S * Hq);
  float* lse2 = ws.take<float>((size_t)S * Hq);
  float *pk = nullptr, *pv = nullptr;
  if (Hq != Hkv) {
    pk = ws.take<float>((size_t)S * Hq * D);
    pv = ws.take<float>((size_t)S * Hq * D);
  }
  if (!ws.ok()) {
    set_error("workspace too small: need %zu bytes, got %zu", ws.used, workspace_bytes);
    return ARTK_ERR_WORKSPACE_TOO_SMALL;
  }
  AttnPlan pl;
  attn_plan_layout(const_cast<void*>(plan), (size_t)1 << 40, S, pl);
  hipStream_t st = (hipStream_t)stream;
  attn_delta_kernel<<<(unsigned)((S * Hq + 15) / 16), 256, 0, st>>>(
      (const uint16_t*)out, strides[6], strides[7], (const uint16_t*)d_out, strides[8], strides[9], lse,
      (int)S, Hq, D, delta, lse2);
  ARTK_CHECK_LAUNCH();
  AttnBwdParams p;
  p.Q = (const uint16_t*)q;
  p.K = (const uint16_t*)k;
  p.V = (const uint16_t*)v;
  p.dO = (const uint16_t*)d_out;
  p.lse2 = lse2;
  p.delta = delta;
  p.dQ = (uint16_t*)dq;
  p.dK = (uint16_t*)dk;
  p.dV = (uint16_t*)dv;
  p.pK = pk;
  p.pV = pv;
  p.q_ss = strides[0];  p.q_hs = strides[1];
  p.k_ss = strides[2];  p.k_hs = strides[3];
  p.v_ss = strides[4];  p.v_hs = strides[5];
  p.do_ss = strides[8]; p.do_hs = strides[9];
  p.dq_ss = strides[10]; p.dq_hs = strides[11];
  p.dk_ss = strides[12]; p.dk_hs = strides[13];
  p.dv_ss = strides[14]; p.dv_hs = strides[15];
  p.gc = pl.gc;
  p.pc = pl.pc;
  p.list = pl.list;
  p.cnt = pl.cnt;
  p.listT = pl.list2;
  p.cntT = pl.cnt2;
  p.S = (int)S;
  p.Hq = Hq;
  p.Hkv = Hkv;
  p.nQb = pl.nQb;
  p.nKb = pl.nKb;
  p.nQb2 = pl.nQb2;
  p.nKb2 = pl.nKb2;
  p.scale = scale;
  p.scale_log2e = scale * LOG2E;
  {
    int cus = 0, dev = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
      cus = 256;
    p.light_max = pl.nKb2 * Hkv >= cus ? ATT_LIGHT_MAX : 0;
    if (g_light_max_override >= 0) p.light_max = g_light_max_override;  // artk_attn_bwd_tuning
  }
  prof_begin(PROF_ATTN_BWD_KV, st);
  if (D == 128)
    attn_bwd_kv_kernel<128><<<(unsigned)(pl.nKb2 * Hq), 512, 0, st>>>(p);
  else
    attn_bwd_kv_kernel<64><<<(unsigned)(pl.nKb2 * Hq), 512, 0, st>>>(p);
  prof_end(PROF_ATTN_BWD_KV, st);
  ARTK_CHECK_LAUNCH();
  if (Hq != Hkv) {
    const int64_t n4 = S * Hkv * (D / 4);
    attn_kv_reduce_kernel<<<(unsigned)((n4 + 255) / 256), 256, 0, st>>>(
        pk, pv, pl.cnt2, p.light_max, Hq / Hkv, S, Hkv, D, scale, (uint16_t*)dk, strides[12], strides[13], (uint16_t*)dv,
        strides[14], strides[15]);
    ARTK_CHECK_LAUNCH();
  }
  prof_begin(PROF_ATTN_BWD_Q, st);
  if (D == 128)
    attn_bwd_dq_kernel<128><<<(unsigned)(pl.nQb * Hq), 512, 0, st>>>(p);
  else
    attn_bwd_dq_kernel<64><<<(unsigned)(pl.nQb * Hq), 512, 0, st>>>(p);
  prof_end(PROF_ATTN_BWD_Q, st);
  ARTK_CHECK_LAUNCH();
  return ARTK_OK;
}

int32_t artk_attn_bwd_tuning(int32_t light_max) {
  g_light_max_override = light_max < 0 ? -1 : light_max;
  return ARTK_OK;
}

}  // extern "C"
