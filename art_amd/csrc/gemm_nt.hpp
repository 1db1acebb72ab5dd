// NT bf16 GEMM main loop for gfx950 (MI355X, CDNA4).
//
// Computes a 256x256 tile of  C[i][j] = sum_k P[i][k] * Q[j][k]  where both
// operands are row-major with K contiguous ("NT").  P is the "row operand"
// (its row index ends up in the accumulator registers of a lane), Q is the
// "column operand" (its row index is the lane's column).  The callers put the
// matrix whose row index is the *contiguous* dimension of the output into the
// P role, so that each lane owns 4 consecutive output elements.
//
// Two work-group shapes share the code, selected by the template parameter NI
// (column-operand MFMA tiles per wavefront):
//   NI = 4: 256 threads = 4 wavefronts in a 2x2 grid, wave tile 128x128 = 4x4
//           MFMA 32x32x16 tiles, 256 fp32 accumulators per lane, 1 wave / SIMD;
//   NI = 2: 512 threads = 8 wavefronts in a 2x4 grid, wave tile 128x64 = 4x2
//           tiles, 128 accumulators per lane, 2 waves / SIMD: while one wave
//           waits (LDS data, a full texture-address FIFO, the barrier, its
//           epilogue) the other keeps the MFMA pipe busy.
// One work-group per CU either way (128 KiB of LDS, all registers).  Measured: NI = 2 is faster for
// every kernel built on this loop once the kernel is persistent (lm_head forward
// +12 %, LoRA GEMMs +7 %, MoE grouped GEMMs +5 %); NI = 4 only won for the
// short-K products while each work-group still paid its own prologue.
//
// Data path: HBM/L2 -> LDS by buffer_load_dwordx4 ... lds (no VGPR staging),
// two LDS stages of 2 x 32 KiB, 16-byte chunks XOR-swizzled so that both the
// DMA writes (1 KiB contiguous per wave instruction) and the ds_read_b128
// operand reads are bank-conflict free.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

namespace artk {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

constexpr int TILE = 256;       // tile rows of either operand
constexpr int BK = 64;          // K elements per LDS stage
template <int NI> constexpr int nthreads() { return 1024 / NI; }   // 256 or 512
constexpr int OPER_STAGE_BYTES = TILE * BK * 2;          // 32 KiB
constexpr int STAGE_BYTES = 2 * OPER_STAGE_BYTES;         // P + Q
constexpr int NSTAGES = 2;
constexpr int GEMM_LDS_BYTES = NSTAGES * STAGE_BYTES;     // 128 KiB

typedef __attribute__((address_space(3))) void* lds_ptr_t;

// Swizzle of the 16-byte chunk index within a 128-byte LDS row.
__device__ __forceinline__ int swz(int row) { return (row & 7) ^ ((row >> 3) & 1); }

// One operand of the NT GEMM as seen by one wavefront's DMA instructions
// (2 * NI instructions of 1 KiB per wave and stage).
template <int NI>
struct OperandLoader {
  static constexpr int DI = 2 * NI;
  __amdgpu_buffer_rsrc_t rsrc;
  int voff[DI];  // per-lane byte offset of the DMA instructions of this wave
  int nlive;     // DMA instructions of this wave that are issued (wave-uniform): DI, or, with
                 // skip_dead, those that carry at least one row of the operand

  // base: first element of the operand; ld: leading dimension in elements;
  // row0: first tile row; nrows: rows the operand really has (rows past the
  // end are clamped to the last valid row; the epilogue never stores them).
  // gather (optional): tile row i reads operand row gather[row0 + i] instead of
  // row0 + i; all gathered rows must lie within 2 GiB of `base`.
  // skip_dead: instructions whose 8 rows all lie past the end are not issued at all; their LDS
  // rows keep whatever an earlier tile left there, so the accumulator columns (or rows) they
  // feed hold garbage, possibly NaN, and the caller must discard them (a partial tile's
  // epilogue does not store them anyway; garbage in one operand row never reaches another).
  __device__ __forceinline__ void init(const void* base, int64_t ld, int64_t row0,
                                       int64_t nrows, int wave, int lane,
                                       const int* gather = nullptr, bool skip_dead = false) {
    const char* p = (const char*)base + (gather ? 0 : row0 * ld * 2);
    rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)p, 0, 0x7fffffff, 0x00020000);
    int64_t left = nrows - row0;
    int nvalid = left >= TILE ? TILE : (int)left;
    int r = lane >> 3, pc = lane & 7;
#pragma unroll
    for (int i = 0; i < DI; ++i) {
      int row = (wave * DI + i) * 8 + r;
      int kc = pc ^ swz(row);
      int64_t rc = row < nvalid ? row : nvalid - 1;
      if (gather) rc = gather[row0 + rc];
      voff[i] = (int)(rc * ld * 2) + kc * 16;
    }
    nlive = DI;
    if (skip_dead) {
      const int live = (nvalid + 7) / 8 - wave * DI;  // instruction j of the tile carries rows 8j .. 8j+7
      nlive = live < 0 ? 0 : (live < DI ? live : DI);
    }
  }

  // Issue DMA instructions LO..HI-1 of this wave's DI for K offset k0 (elements)
  // into the 32 KiB operand stage at `stage` (LDS byte address, wave-uniform).
  // DMA instruction i alone (i a compile-time constant at every call site).
  __device__ __forceinline__ void issue_one(char* stage, int wave, int k0, int i) const {
    if (i < nlive)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lds_ptr_t)(stage + (wave * DI + i) * 1024), 16, voff[i],
                                               k0 * 2, 0, 0);
  }
  // (TAG is unused: callers that are themselves instantiated several times pass a distinct value each)
  template <int LO, int HI, int TAG = 0>
  __device__ __forceinline__ void issue(char* stage, int wave, int k0) const {
#pragma unroll
    for (int i = LO; i < HI; ++i) {
      if (i < nlive)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lds_ptr_t)(stage + (wave * DI + i) * 1024), 16,
                                                 voff[i], k0 * 2, 0, 0);
    }
  }
};

template <int NI>
struct TileAcc {
  floatx16 c[4][NI];  // [mi][ni]
  __device__ __forceinline__ void zero() {
#pragma unroll
    for (int mi = 0; mi < 4; ++mi)
#pragma unroll
      for (int ni = 0; ni < NI; ++ni)
#pragma unroll
        for (int j = 0; j < 16; ++j) c[mi][ni][j] = 0.f;
  }
};

// Row (P-operand index, tile-relative) of accumulator element j of MFMA tile mi
// for this lane: wm * 128 + mi * 32 + (j / 4) * 8 + (lane / 32) * 4 + j % 4;
// column (Q-operand index, tile-relative) of MFMA tile ni:
template <int NI>
__device__ __forceinline__ int acc_col(int wn, int ni, int lane) {
  return wn * (32 * NI) + ni * 32 + (lane & 31);
}
// Position of a wavefront in the 2 (row operand) x (8 / NI) (column operand) grid.
template <int NI> __device__ __forceinline__ int wave_m(int wave) { return wave / (8 / NI); }
template <int NI> __device__ __forceinline__ int wave_n(int wave) { return wave % (8 / NI); }

// Operand fragments of one K=16 step: 4 row-operand and NI column-operand reads.
template <int NI>
struct Frags {
  bf16x8 p[4], q[NI];
};

// NQ (<= NI): column-operand tiles of this wave that are computed; the others are left alone
// (a partial tile whose last columns nobody stores).  NQ = 0: nothing is read or multiplied.
template <int NI, int NQ = NI>
__device__ __forceinline__ void load_frags(Frags<NI>& f, const char* sp, const char* sq, int off) {
  if constexpr (NQ > 0) {
#pragma unroll
    for (int mi = 0; mi < 4; ++mi) f.p[mi] = *(const bf16x8*)(sp + off + mi * 4096);
#pragma unroll
    for (int ni = 0; ni < NQ; ++ni) f.q[ni] = *(const bf16x8*)(sq + off + ni * 4096);
  }
}

template <int NI, int NQ = NI>
__device__ __forceinline__ void mma_frags(TileAcc<NI>& acc, const Frags<NI>& f) {
#pragma unroll
  for (int mi = 0; mi < 4; ++mi)
#pragma unroll
    for (int ni = 0; ni < NQ; ++ni)
      acc.c[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f.p[mi], f.q[ni], acc.c[mi][ni], 0, 0, 0);
}

// bf16 store of one 32x32 accumulator block whose 32 rows are contiguous in the
// output (dst = this lane's column, block row 0; 16-byte aligned).  Lanes l and
// l + 32 hold the same column, each 4 rows of every 8.  They trade halves
// (v_permlane32_swap), so that every lane stores 8 consecutive rows as 16 bytes:
// rows 16p .. 16p+7 from the lower lane, 16p+8 .. 16p+15 from the upper one, and a
// store instruction puts down 32 contiguous bytes per column instead of 16.
// Both lanes of a pair must call it together.
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2_t;
  bf16x2_t v = {(__bf16)lo, (__bf16)hi};
  return *(uint32_t*)&v;
}
__device__ __forceinline__ void store_block_bf16(uint16_t* dst, const floatx16& c, int half) {
#pragma unroll
  for (int p = 0; p < 2; ++p) {
    const uint32_t a0 = pack_bf16x2(c[8 * p + 0], c[8 * p + 1]), a1 = pack_bf16x2(c[8 * p + 2], c[8 * p + 3]);
    const uint32_t b0 = pack_bf16x2(c[8 * p + 4], c[8 * p + 5]), b1 = pack_bf16x2(c[8 * p + 6], c[8 * p + 7]);
    // swap(a, b): a' = {lower lanes: own a, upper lanes: the lower lane's b},
    //             b' = {lower lanes: the upper lane's a, upper lanes: own b}
    const auto r0 = __builtin_amdgcn_permlane32_swap(a0, b0, false, false);
    const auto r1 = __builtin_amdgcn_permlane32_swap(a1, b1, false, false);
    const uint4 v = {r0[0], r1[0], r0[1], r1[1]};
    *(uint4*)(dst + 16 * p + 8 * half) = v;
  }
}

// LDS scratch of an epilogue that transposes a wave's 128 x 64 block (8-wave shape) 32 columns
// at a time: 32 rows of 256 bytes at a pitch of 272 per wave (8-byte writes down a column and
// 16-byte reads along a row are then free of bank conflicts).  Eight of them cover the second
// GEMM stage, which is idle during an epilogue (the next tile's first DMA stage only fills the
// first), plus EPI_LDS_EXTRA bytes behind it.
constexpr int EPI_PITCH = 272;
constexpr int EPI_LDS_PER_WAVE = 32 * EPI_PITCH;                   // 8704
constexpr int EPI_LDS_EXTRA = 8 * EPI_LDS_PER_WAVE - STAGE_BYTES;  // 4096

// The two operand loaders and the K range of one tile.  Separate from the main
// loop so that a kernel that walks several tiles can set up the next tile's
// loaders and start its first DMA stage before the current tile's epilogue
// (its prologue latency then hides behind that epilogue).
template <int NI>
struct TileLoaders {
  OperandLoader<NI> lp, lq;
  int k_begin, k_end;
  __device__ __forceinline__ void init(const void* P, int64_t ldp, int64_t prow0, int64_t prows,
                                       const void* Q, int64_t ldq, int64_t qrow0, int64_t qrows, int kb,
                                       int ke, const int* qgather = nullptr, bool q_skip_dead = false) {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    lp.init(P, ldp, prow0, prows, wave, lane);
    lq.init(Q, ldq, qrow0, qrows, wave, lane, qgather, q_skip_dead);
    k_begin = kb;
    k_end = ke;
  }
  // DMA instructions LO .. HI-1 of this wave's share of both operands, K offset k0, into the stage at
  // `stage`.  (TAG is unused: callers that are themselves instantiated several times pass a distinct
  // value each.)
  template <int LO, int HI, int TAG>
  __device__ __forceinline__ void issue(char* stage, int wave, int k0) const {
    lp.template issue<LO, HI, TAG>(stage, wave, k0);
    lq.template issue<LO, HI, TAG>(stage + OPER_STAGE_BYTES, wave, k0);
  }
  // DMA instructions that issue<LO, LO + 1> stands for (the instruction order is pinned with it).
  static constexpr int DMA_PER_INDEX = 2;
  // First K stage into LDS stage 0.  No wave of the work-group may still be
  // reading stage 0 (true at kernel start and after gemm_tile_run returns).
  __device__ __forceinline__ void issue_first(char* smem) const {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    issue<0, 2 * NI, 77>(smem, wave, k_begin);
  }
};

// Main loop over the K range of L (L.issue_first(smem) must have been called by
// every wave): acc += P[prow0 : prow0+256, k_begin : k_end] * Q[qrow0 : qrow0+256, same]^T.
// k_begin/k_end are multiples of BK, k_end > k_begin.  `smem` is GEMM_LDS_BYTES
// of LDS, 1 KiB aligned.
//
// Schedule of one K-step (BK = 64 = 4 MFMA steps of K = 16, 8 MFMAs each per wave):
//   steps 0..2 : MFMAs of step kk while the fragments of step kk+1 are read;
//                the second half of the DMA for the next stage is issued here
//   wait for own LDS reads and own DMA, barrier:
//                every wave holds its step-3 fragments in registers, so the
//                current stage is free, and the next stage has landed
//   step 3     : MFMAs while step 0 of the next stage is read; the first half
//                of the DMA for the stage after next goes into the freed buffer
// The loop body has no branches; the last two K-steps are peeled off without the DMA
// that would reach past the end of the K range.
__device__ __forceinline__ void gemm_tile_run_pinned(TileAcc<4>& acc, char* smem, const TileLoaders<4>& L);
template <int NQ, bool ALL_EARLY, class LOADERS>
__device__ __forceinline__ void gemm_tile_run_8(TileAcc<2>& acc, char* smem, const LOADERS& L,
                                                std::integral_constant<int, NQ>,
                                                std::integral_constant<bool, ALL_EARLY>);

// Instruction-order group: one MFMA, then N DMA issues, then one LDS read.
template <int N>
__device__ __forceinline__ void mfma_dma_read_group() {
  __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
  if constexpr (N > 0) __builtin_amdgcn_sched_group_barrier(0x020, N, 0);
  __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
}

template <int NI, int NQ = NI, bool ALL_EARLY = false, class LOADERS = TileLoaders<NI>>
__device__ __forceinline__ void gemm_tile_run(TileAcc<NI>& acc, char* smem, const LOADERS& L) {
  if constexpr (NI == 4) {
    gemm_tile_run_pinned(acc, smem, L);  // one wave per SIMD: the order is pinned (see below)
    return;
  } else {
    gemm_tile_run_8(acc, smem, L, std::integral_constant<int, NQ>{}, std::integral_constant<bool, ALL_EARLY>{});
  }
}
template <int NQ, bool ALL_EARLY, class LOADERS>
__device__ __forceinline__ void gemm_tile_run_8(TileAcc<2>& acc, char* smem, const LOADERS& L,
                                                std::integral_constant<int, NQ>,
                                                std::integral_constant<bool, ALL_EARLY>) {
  constexpr int NI = 2;
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int wm = wave_m<NI>(wave), wn = wave_n<NI>(wave);
  constexpr int DI = 2 * NI;
  const int k_begin = L.k_begin, k_end = L.k_end;

  // Per-lane LDS read offsets (within an operand stage) for the 4 K=16 steps.
  int off[4];
  {
    int rl = lane & 31;
    int f = swz(rl);
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) off[kk] = rl * 128 + (((kk * 2 + (lane >> 5)) ^ f) << 4);
  }
  const int p_wave_off = wm * 128 * 128;
  const int q_wave_off = OPER_STAGE_BYTES + wn * (32 * NI) * 128;

  const int nk = (k_end - k_begin) / BK;

  // DMA instructions per operand issued right after the barrier that frees their buffer, the rest at the
  // start of the next K-step.  All of them early (a full K-step of lead) pays where most row-operand
  // panels miss in L2 (grouped GEMMs whose weights serve two or three tiles: +1-2 %); elsewhere the split
  // is faster (lm_head forward at a hidden size of 896: 6 %, LoRA linear: 1.4 %).
  constexpr int EARLY = ALL_EARLY ? DI : NI;
  constexpr int TG = NQ + (ALL_EARLY ? 10 : 0);  // issue<> tag
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  if (nk > 1) {
    L.template issue<0, EARLY, TG>(smem + STAGE_BYTES, wave, k_begin + BK);
  }
  Frags<NI> f0, f1;
  load_frags<NI, NQ>(f0, smem + p_wave_off, smem + q_wave_off, off[0]);

  // One K-step.  LATE: the second half of stage kt + 1 is still to be issued (false in the last
  // K-step); AHEAD: the first half of stage kt + 2 goes out after the barrier (false in the last
  // two).  The last K-steps are peeled off with those flags cleared instead of re-fetching the
  // last stage: on a 12-step K loop the re-fetches were an eighth of the traffic into LDS.
  auto k_step = [&](int kt, auto late_tag, auto ahead_tag) {
    constexpr bool LATE = decltype(late_tag)::value, AHEAD = decltype(ahead_tag)::value;
    char* cur = smem + (kt & 1) * STAGE_BYTES;
    char* nxt = smem + ((kt + 1) & 1) * STAGE_BYTES;
    const char* sp = cur + p_wave_off;
    const char* sq = cur + q_wave_off;

    if constexpr (LATE) {
      const int k1 = k_begin + (kt + 1) * BK;
      L.template issue<EARLY, DI, TG + 100>(nxt, wave, k1);
    }
    load_frags<NI, NQ>(f1, sp, sq, off[1]);
    mma_frags<NI, NQ>(acc, f0);
    load_frags<NI, NQ>(f0, sp, sq, off[2]);
    mma_frags<NI, NQ>(acc, f1);
    load_frags<NI, NQ>(f1, sp, sq, off[3]);
    mma_frags<NI, NQ>(acc, f0);
    // Interleave: 3 steps of 4*NI MFMAs, 3*(4+NI) LDS reads, NLATE DMA issues.
    constexpr int NLATE = LATE ? LOADERS::DMA_PER_INDEX * (DI - EARLY) : 0;
    if constexpr (NI == 4) {
#pragma unroll
      for (int i = 0; i < NLATE; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);  // 2 MFMA
        __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);  // 1 DMA issue
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // 1 LDS read
      }
#pragma unroll
      for (int i = 0; i < 24 - NLATE; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
    } else {
#pragma unroll
      for (int i = 0; i < NLATE; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // 1 MFMA
        __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);  // 1 DMA issue
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // 1 LDS read
      }
#pragma unroll
      for (int i = 0; i < 18 - NLATE; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, 6, 0);
    }

    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    __syncthreads();

    if constexpr (AHEAD) {
      const int k2 = k_begin + (kt + 2) * BK;
      L.template issue<0, EARLY, TG + 200>(cur, wave, k2);
    }
    // (after the last K-step this reads the idle stage: values nobody uses)
    load_frags<NI, NQ>(f0, nxt + p_wave_off, nxt + q_wave_off, off[0]);
    mma_frags<NI, NQ>(acc, f1);
    // 4*NI MFMA, 4+NI LDS reads, NA DMA issues
    if constexpr (NI == 4) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
        if (AHEAD && i < EARLY) __builtin_amdgcn_sched_group_barrier(0x020, 2, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
    } else {
      constexpr int NA = AHEAD ? LOADERS::DMA_PER_INDEX * EARLY : 0;  // spread over the six groups
      mfma_dma_read_group<NA / 6 + (0 < NA % 6)>();
      mfma_dma_read_group<NA / 6 + (1 < NA % 6)>();
      mfma_dma_read_group<NA / 6 + (2 < NA % 6)>();
      mfma_dma_read_group<NA / 6 + (3 < NA % 6)>();
      mfma_dma_read_group<NA / 6 + (4 < NA % 6)>();
      mfma_dma_read_group<NA / 6 + (5 < NA % 6)>();
      __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
    }
  };
  using yes = std::integral_constant<bool, true>;
  using no = std::integral_constant<bool, false>;
  for (int kt = 0; kt < nk - 2; ++kt) k_step(kt, yes{}, yes{});
  if (nk > 1) k_step(nk - 2, yes{}, no{});
  k_step(nk - 1, no{}, no{});
  // Nothing is outstanding here; the caller may reuse or release LDS.
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
  __syncthreads();
}

// gemm_tile_run for a tile whose column operand has only `ncols` (<= 256) rows that anybody
// stores: a wave computes only those of its NI 32-column tiles that contain such a column
// (wave-uniform choice; every variant executes the same barriers).  8-wave shape only.  Its caller
// is the grouped GEMM, so the whole fill of a stage is requested right after the barrier.
__device__ __forceinline__ void gemm_tile_run_cols(TileAcc<2>& acc, char* smem, const TileLoaders<2>& L,
                                                   int ncols) {
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int left = ncols - wave_n<2>(wave) * 64;  // columns of this wave that are stored
  if (left > 32) gemm_tile_run<2, 2, true>(acc, smem, L);
  else if (left > 0) gemm_tile_run<2, 1, true>(acc, smem, L);
  else gemm_tile_run<2, 0, true>(acc, smem, L);
}

// ----------------------------------------------------------------------------
// Main loop for the 4-wave shape (NI = 4) with the instruction order pinned.
//
// One wave per SIMD means nothing hides a stall: an LDS read that is waited for
// right after it was issued, or MFMAs bunched behind a row of reads, idle the
// matrix pipe for the whole latency.  Left to itself the scheduler sinks the
// fragment reads of step kk+1 down to their first use.  Here every K = 16 step is
// written as 8 groups of {2 MFMAs of step kk, 1 fragment read of step kk+1, at most
// one DMA instruction}, with a scheduling barrier after each group, so the reads
// of a step are issued 256 .. 512 MFMA cycles before their first use and the
// compiler's own s_waitcnt placement (it counts the reads in order) never blocks.
// Same stages, barrier and DMA split as gemm_tile_run.  Measured on 5632 x 152064
// x 3584: the matrix pipe is busy 87 % of the main loop's cycles (HIP cycle counter
// against the constant-rate counter: the clock settles near 1.6 GHz under this load).
// ----------------------------------------------------------------------------
struct Frags4 {
  bf16x8 p[4], q[4];
};

// Fragment G of a step's read order p0 q0 q1 q2 q3 p1 p2 p3, from the operand stages at (sp, sq).
template <int G>
__device__ __forceinline__ void read_frag4(Frags4& f, const char* sp, const char* sq, int off) {
  constexpr bool is_q = G >= 1 && G <= 4;
  constexpr int idx = G == 0 ? 0 : is_q ? G - 1 : G - 4;
  if constexpr (is_q) f.q[idx] = *(const bf16x8*)(sq + off + idx * 4096);
  else f.p[idx] = *(const bf16x8*)(sp + off + idx * 4096);
}

// The two MFMAs of group G of a step.  The 16 tiles are walked in a serpentine (row 0 left
// to right, row 1 right to left, ...): the fragments that are read first are used first.
// (Other orders, also one that accumulates K = 32 into a tile before moving on, measure the same.)
template <int G>
__device__ __forceinline__ void mma_group4(TileAcc<4>& acc, const Frags4& f) {
  constexpr int m = G / 2;
  constexpr int na = (m & 1) ? 3 - 2 * (G & 1) : 2 * (G & 1);
  constexpr int nb = (m & 1) ? na - 1 : na + 1;
  acc.c[m][na] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f.p[m], f.q[na], acc.c[m][na], 0, 0, 0);
  acc.c[m][nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f.p[m], f.q[nb], acc.c[m][nb], 0, 0, 0);
}

// Group G of a step: its two MFMAs on `use`, fragment G of the following step into
// `fill`, and DMA instruction D of this wave (0..7: row operand, 8..15: column
// operand; -1: none) into the stage at `dst` for K offset k.
template <int G, int D>
__device__ __forceinline__ void pinned_group(TileAcc<4>& acc, const Frags4& use, Frags4& fill, const char* sp,
                                             const char* sq, int off, const OperandLoader<4>& lp,
                                             const OperandLoader<4>& lq, char* dst, int wave, int k) {
  mma_group4<G>(acc, use);
  read_frag4<G>(fill, sp, sq, off);
  if constexpr (D >= 0 && D < 8) lp.issue_one(dst, wave, k, D);
  if constexpr (D >= 8) lq.issue_one(dst + OPER_STAGE_BYTES, wave, k, D - 8);
  __builtin_amdgcn_sched_barrier(0);
}

// One K = 16 step; D0 >= 0: DMA instructions D0 .. D0+3 of each operand ride in its 8 groups.
template <int D0>
__device__ __forceinline__ void pinned_step(TileAcc<4>& acc, const Frags4& use, Frags4& fill, const char* sp,
                                            const char* sq, int off, const OperandLoader<4>& lp,
                                            const OperandLoader<4>& lq, char* dst, int wave, int k) {
  constexpr bool dma = D0 >= 0;
  pinned_group<0, dma ? D0 + 0 : -1>(acc, use, fill, sp, sq, off, lp, lq, dst, wave, k);
  pinned_group<1, dma ? D0 + 8 : -1>(acc, use, fill, sp, sq, off, lp, lq, dst, wave, k);
  pinned_group<2, dma ? D0 + 1 : -1>(acc, use, fill, sp, sq, off, lp, lq, dst, wave, k);
  pinned_group<3, dma ? D0 + 9 : -1>(acc, use, fill, sp, sq, off, lp, lq, dst, wave, k);
  pinned_group<4, dma ? D0 + 2 : -1>(acc, use, fill, sp, sq, off, lp, lq, dst, wave, k);
  pinned_group<5, dma ? D0 + 10 : -1>(acc, use, fill, sp, sq, off, lp, lq, dst, wave, k);
  pinned_group<6, dma ? D0 + 3 : -1>(acc, use, fill, sp, sq, off, lp, lq, dst, wave, k);
  pinned_group<7, dma ? D0 + 11 : -1>(acc, use, fill, sp, sq, off, lp, lq, dst, wave, k);
}

__device__ __forceinline__ void gemm_tile_run_pinned(TileAcc<4>& acc, char* smem, const TileLoaders<4>& L) {
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int wm = wave_m<4>(wave), wn = wave_n<4>(wave);
  const OperandLoader<4>& lp = L.lp;
  const OperandLoader<4>& lq = L.lq;
  const int k_begin = L.k_begin, k_end = L.k_end;
  int off[4];
  {
    int rl = lane & 31;
    int f = swz(rl);
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) off[kk] = rl * 128 + (((kk * 2 + (lane >> 5)) ^ f) << 4);
  }
  const int p_wave_off = wm * 128 * 128;
  const int q_wave_off = OPER_STAGE_BYTES + wn * 128 * 128;
  const int nk = (k_end - k_begin) / BK;
  const int k_last = k_end - BK;

  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  Frags4 fa, fb;
  {
    // fragments of step 0 of the first stage; first half of the second stage's DMA
    const char* sp = smem + p_wave_off;
    const char* sq = smem + q_wave_off;
    read_frag4<0>(fa, sp, sq, off[0]);
    read_frag4<1>(fa, sp, sq, off[0]);
    read_frag4<2>(fa, sp, sq, off[0]);
    read_frag4<3>(fa, sp, sq, off[0]);
    read_frag4<4>(fa, sp, sq, off[0]);
    read_frag4<5>(fa, sp, sq, off[0]);
    read_frag4<6>(fa, sp, sq, off[0]);
    read_frag4<7>(fa, sp, sq, off[0]);
    int k1 = k_begin + BK < k_last ? k_begin + BK : k_last;
#pragma unroll
    for (int i = 0; i < 4; ++i) lp.issue_one(smem + STAGE_BYTES, wave, k1, i);
#pragma unroll
    for (int i = 0; i < 4; ++i) lq.issue_one(smem + STAGE_BYTES + OPER_STAGE_BYTES, wave, k1, i);
    __builtin_amdgcn_sched_barrier(0);
  }
  for (int kt = 0; kt < nk; ++kt) {
    char* cur = smem + (kt & 1) * STAGE_BYTES;
    char* nxt = smem + ((kt + 1) & 1) * STAGE_BYTES;
    const char* sp = cur + p_wave_off;
    const char* sq = cur + q_wave_off;
    int k1 = k_begin + (kt + 1) * BK;
    k1 = k1 < k_last ? k1 : k_last;
    // steps 0..2 of this stage; the second half of the next stage's DMA rides in step 0
    pinned_step<4>(acc, fa, fb, sp, sq, off[1], lp, lq, nxt, wave, k1);
    pinned_step<-1>(acc, fb, fa, sp, sq, off[2], lp, lq, nxt, wave, k1);
    pinned_step<-1>(acc, fa, fb, sp, sq, off[3], lp, lq, nxt, wave, k1);
    // fb holds step 3: the current stage is free once every wave is here, and the next has landed
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    int k2 = k_begin + (kt + 2) * BK;
    k2 = k2 < k_last ? k2 : k_last;
    // step 3: MFMAs while step 0 of the next stage is read; first half of the DMA for the
    // stage after next goes into the freed buffer
    pinned_step<0>(acc, fb, fa, nxt + p_wave_off, nxt + q_wave_off, off[0], lp, lq, cur, wave, k2);
  }
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
  __syncthreads();
}

template <int NI>
__device__ __forceinline__ void gemm_tile_nt(TileAcc<NI>& acc, char* smem, const void* P, int64_t ldp,
                                             int64_t prow0, int64_t prows, const void* Q,
                                             int64_t ldq, int64_t qrow0, int64_t qrows, int k_begin,
                                             int k_end, const int* qgather = nullptr) {
  TileLoaders<NI> L;
  L.init(P, ldp, prow0, prows, Q, ldq, qrow0, qrows, k_begin, k_end, qgather);
  L.issue_first(smem);
  gemm_tile_run(acc, smem, L);
}

// Map the hardware's round-robin block->XCD placement (block b runs on XCD
// b % 8) onto contiguous ranges of logical tile ids, so that tiles sharing
// operand panels run on the same XCD and hit in its private L2.
__device__ __forceinline__ int xcd_remap(int bid, int nblocks) {
  int full = nblocks >> 3, rem = nblocks & 7;
  int x = bid & 7, loc = bid >> 3;
  int start = x * full + (x < rem ? x : rem);
  return start + loc;
}


// Logical tile id -> (row-operand tile, column-operand tile).  Ids walk down a
// group of `group` row-operand tiles before moving to the next column-operand
// tile, so the 32 work-groups that run together on one XCD cover a group x
// (32/group) patch and share operand panels in that XCD's L2.  Which split of the
// 32 is best depends on where the operands come from: a patch fetches `group`
// row-operand panels and 32/group column-operand panels per K step, and a panel of
// a small operand that every XCD keeps re-reading (the hidden states of a chunk,
// the activations of a layer) is served by the Infinity Cache, while the panels of
// a large streaming operand (the 1.1 GB lm_head) come from HBM the first time.
// Measured on 152064 x 5632 x 3584 (lm_head forward): group 4 gives 1290 TFLOP/s,
// 3 / 5 / 6: 1255, 8: 1222, 2: 1240, 16: 1105; on 22016 x 8192 x 2048 (LoRA
// gate|up, both operands resident): 8 gives 1225, 4 and 16: 1160, 2: 1070.
constexpr int TILE_GROUP = 8;
constexpr int TILE_GROUP_STREAMING = 4;  // row operand streams from HBM, column operand is small
__device__ __forceinline__ void tile_coords(int id, int row_tiles, int col_tiles, int& rt, int& ct,
                                            int group = TILE_GROUP) {
  const int per = group * col_tiles;
  const int g = id / per;
  const int first = g * group;
  const int gs = row_tiles - first < group ? row_tiles - first : group;
  const int w = id - g * per;
  rt = first + w % gs;
  ct = w / gs;
}

}  // namespace artk
