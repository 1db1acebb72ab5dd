// NT bf16 GEMM main loop for gfx950, half-width shape: a 256 x 128 tile per work-group of
// 4 wavefronts (2 x 2, wave tile 128 x 64 = 4 x 2 MFMA 32x32x16 tiles, the same wave tile as
// the 8-wave shape of gemm_nt.hpp), sized so that TWO work-groups share a CU: 128 accumulators
// + fragments fit the 256 registers a wave has at two waves per SIMD, and the LDS ring is
// 3 stages of K = 32 (24 KiB each, 72 KiB per work-group).
//
// Why: the two work-groups of a CU run independent tiles with independent barriers, so while
// one of them sits in its epilogue, its prologue, a barrier or a cache miss, the other one's
// wave on the same SIMD has the matrix pipe to itself.  With one work-group per CU all waves
// reach the epilogue together and the pipe idles for its whole length; on short K loops (a
// 14-step loop per tile for a hidden size of 896) that idle time is as long as the loop.
// The price is 1.5 x the traffic into LDS per flop (the 256-row operand is fetched once per
// 128 columns instead of once per 256), which long K loops at the power limit do not repay.
//
// Data path and swizzle as in gemm_nt.hpp, with 64-byte LDS rows (K = 32): a row's four
// 16-byte chunks are XOR-ed with (row / 4) % 4, which makes the 1 KiB DMA writes (16 rows per
// instruction) and the ds_read_b128 fragment reads (rows r .. r + 15 of one chunk column)
// bank-conflict free.
#pragma once
#include "gemm_nt.hpp"

namespace artk {

constexpr int HALF_Q = 128;                               // column-operand rows per tile
constexpr int HBK = 32;                                   // K elements per LDS stage
constexpr int HALF_P_STAGE = TILE * HBK * 2;              // 16 KiB
constexpr int HALF_Q_STAGE = HALF_Q * HBK * 2;            // 8 KiB
constexpr int HALF_STAGE = HALF_P_STAGE + HALF_Q_STAGE;   // 24 KiB
constexpr int HALF_NSTAGES = 3;
constexpr int HALF_LDS_BYTES = HALF_NSTAGES * HALF_STAGE; // 72 KiB
constexpr int HALF_THREADS = 256;

__device__ __forceinline__ int hswz(int row) { return (row >> 2) & 3; }

// Both operands of one tile as seen by one wavefront's DMA instructions: 4 of the row
// operand's 16 and 2 of the column operand's 8 per stage (1 KiB = 16 rows of 64 bytes each).
struct HalfLoaders {
  __amdgpu_buffer_rsrc_t rp, rq;
  int vp[4], vq[2];
  int k_begin, k_end;

  // P: row operand [prows, ldp], tile rows prow0 .. +255; Q: column operand, tile rows
  // qrow0 .. +127 (rows past the end are clamped to the last one; the epilogue never stores
  // them).  qgather (optional): tile row i of Q reads row qgather[qrow0 + i].
  __device__ __forceinline__ void init(const void* P, int64_t ldp, int64_t prow0, int64_t prows, const void* Q,
                                       int64_t ldq, int64_t qrow0, int64_t qrows, int kb, int ke,
                                       const int* qgather = nullptr) {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    const int r = lane >> 2, pc = lane & 3;
    rp = __builtin_amdgcn_make_buffer_rsrc((void*)((const char*)P + prow0 * ldp * 2), 0, 0x7fffffff, 0x00020000);
    rq = __builtin_amdgcn_make_buffer_rsrc((void*)((const char*)Q + (qgather ? 0 : qrow0 * ldq * 2)), 0,
                                           0x7fffffff, 0x00020000);
    const int64_t pleft = prows - prow0, qleft = qrows - qrow0;
    const int pvalid = pleft >= TILE ? TILE : (int)pleft;
    const int qvalid = qleft >= HALF_Q ? HALF_Q : (int)qleft;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int row = (wave * 4 + i) * 16 + r;
      const int64_t rc = row < pvalid ? row : pvalid - 1;
      vp[i] = (int)(rc * ldp * 2) + ((pc ^ hswz(row)) << 4);
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int row = (wave * 2 + i) * 16 + r;
      int64_t rc = row < qvalid ? row : qvalid - 1;
      if (qgather) rc = qgather[qrow0 + rc];
      vq[i] = (int)(rc * ldq * 2) + ((pc ^ hswz(row)) << 4);
    }
    k_begin = kb;
    k_end = ke;
  }

  // The 6 DMA instructions of this wave for K offset k0 into the 24 KiB stage at `stage`.
  // (TAG is unused: it keeps the instantiations of different call sites apart.)
  template <int TAG>
  __device__ __forceinline__ void issue_stage(char* stage, int wave, int k0) const {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rp, (lds_ptr_t)(stage + (wave * 4 + i) * 1024), 16, vp[i], k0 * 2, 0,
                                               0);
#pragma unroll
    for (int i = 0; i < 2; ++i)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rq, (lds_ptr_t)(stage + HALF_P_STAGE + (wave * 2 + i) * 1024), 16,
                                               vq[i], k0 * 2, 0, 0);
  }

  // First two K stages into ring slots 0 and 1.  No wave of the work-group may still be
  // reading the ring (true at kernel start and after gemm_half_run returns).
  __device__ __forceinline__ void issue_first(char* smem) const {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    issue_stage<90>(smem, wave, k_begin);
    if (k_end - k_begin > HBK) issue_stage<91>(smem + HALF_STAGE, wave, k_begin + HBK);
  }
};

__device__ __forceinline__ void load_frags_half(Frags<2>& f, const char* sp, const char* sq, int off) {
#pragma unroll
  for (int mi = 0; mi < 4; ++mi) f.p[mi] = *(const bf16x8*)(sp + off + mi * 2048);
#pragma unroll
  for (int ni = 0; ni < 2; ++ni) f.q[ni] = *(const bf16x8*)(sq + off + ni * 2048);
}

// acc += P[prow0 : +256, k_begin : k_end] * Q[qrow0 : +128, same]^T  (L.issue_first(smem) already
// called by every wave; k_begin / k_end multiples of HBK, k_end > k_begin; smem: HALF_LDS_BYTES,
// 1 KiB aligned).  Accumulator layout: TileAcc<2> with wm = wave / 2, wn = wave % 2:
// row wm*128 + mi*32 + (j/4)*8 + (lane/32)*4 + j%4, column wn*64 + ni*32 + lane%32.
//
// One K = 32 step: the stage after next is requested (its slot was released by the barrier that
// ended the previous step), the second half's fragments are read while the first half
// multiplies; then the wave waits for its own share of the next stage (the 6 newest DMA
// instructions may still be in flight: loads complete in order) and the barrier makes the
// next stage visible and the current one free; the first fragments of the next stage are read
// while the second half multiplies.
__device__ __forceinline__ void gemm_half_run(TileAcc<2>& acc, char* smem, const HalfLoaders& L) {
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int wm = wave >> 1, wn = wave & 1;
  int off[2];
  {
    const int rl = lane & 31;
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) off[kk] = rl * 64 + (((kk * 2 + (lane >> 5)) ^ hswz(rl)) << 4);
  }
  const int p_wave_off = wm * 128 * 64;
  const int q_wave_off = HALF_P_STAGE + wn * 64 * 64;
  const int nk = (L.k_end - L.k_begin) / HBK;

  // also covers the previous tile's stores, which were issued after this tile's first stages
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  char* cur = smem;
  char* nxt = smem + HALF_STAGE;
  char* fil = smem + 2 * HALF_STAGE;
  Frags<2> f0, f1;
  load_frags_half(f0, cur + p_wave_off, cur + q_wave_off, off[0]);

  auto k_step = [&](int kt, auto fill_tag) {
    constexpr bool FILL = decltype(fill_tag)::value;  // stage kt + 2 exists
    if constexpr (FILL) L.issue_stage<FILL ? 92 : 93>(fil, wave, L.k_begin + (kt + 2) * HBK);
    load_frags_half(f1, cur + p_wave_off, cur + q_wave_off, off[1]);
    mma_frags<2, 2>(acc, f0);
#pragma unroll
    for (int i = 0; i < 6; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);             // 1 MFMA
      if (FILL) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);   // 1 DMA issue
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);             // 1 LDS read
    }
    __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
    if constexpr (FILL) asm volatile("s_waitcnt vmcnt(6) lgkmcnt(0)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    __syncthreads();
    // (after the last step this reads a slot nobody filled: values nobody uses)
    load_frags_half(f0, nxt + p_wave_off, nxt + q_wave_off, off[0]);
    mma_frags<2, 2>(acc, f1);
#pragma unroll
    for (int i = 0; i < 6; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
    char* t = cur;
    cur = nxt;
    nxt = fil;
    fil = t;
  };
  using yes = std::integral_constant<bool, true>;
  using no = std::integral_constant<bool, false>;
  for (int kt = 0; kt < nk - 2; ++kt) k_step(kt, yes{});
  if (nk > 1) k_step(nk - 2, no{});
  k_step(nk - 1, no{});
  // Nothing is outstanding here; the caller may refill the ring.
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
  __syncthreads();
}

}  // namespace artk
