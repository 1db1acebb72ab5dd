// 8-wave NT bf16 main loop for two operands WITHOUT row gather (see gemm_nt.hpp for the tile, the
// LDS stages, the swizzle and the loop itself, which are the same), with a change to who issues
// the L2 -> LDS DMA:
//
// The first wave of each SIMD issues the DMA of both.  With two waves per SIMD the older wave
// wins the matrix pipe whenever both have an MFMA ready; it runs ahead and then sits at the
// K-step's barrier (about 900 of 2550 cycles) while the younger one catches up.  Every issue
// slot the younger wave spends on DMA instructions there delays the barrier for everybody; the
// older wave's are free.  So waves 0..3 issue their own share of a stage and that of wave + 4,
// and waves 4..7 run a copy of the loop without any DMA (one wave-uniform branch around the
// whole K loop: a condition around every DMA instruction would become a scalar branch each
// and cut the K-step into basic blocks, across which the instruction order cannot be pinned;
// switching the lanes off around each instruction costs more than it saves, 1140 against 1300
// TFLOP/s on the lm_head shape).
//
// That costs no registers: the tile rows of a plain operand are consecutive rows of the matrix,
// so the 32 DMA instructions of an operand stage (8 rows of 128 bytes each) differ only by a
// multiple of 8 * ld * 2 bytes, which goes into the scalar offset, and a lane keeps two offsets
// per operand (the swizzle alternates with the parity of the instruction).  Rows past the end
// of the operand are out of range of the buffer resource and arrive as zeros (on gfx950 the
// range check covers the scalar offset, and out-of-range lanes of a DMA write zeros to LDS).
#pragma once
#include "gemm_nt.hpp"

namespace artk {

// Whether this wave is one of the four that issue the DMA (wave-uniform).
__device__ __forceinline__ bool plain8_leader() { return __builtin_amdgcn_readfirstlane(threadIdx.x >> 6) < 4; }

struct PanelLoader {
  __amdgpu_buffer_rsrc_t rsrc;  // base: first row of the tile; size: the tile's valid rows
  int voff[2];                  // per-lane byte offset inside an 8-row group [group parity]
  int step;                     // bytes between 8-row groups

  __device__ __forceinline__ void init(const void* base, int64_t ld, int64_t row0, int64_t nrows, int lane) {
    const char* p = (const char*)base + row0 * ld * 2;
    const int64_t left = nrows - row0;
    const int64_t nvalid = left >= TILE ? TILE : (left > 0 ? left : 0);
    // (a tile spans 256 * ld * 2 bytes, which must stay below 2 GiB as for every loader here: the
    // per-lane offsets are 32-bit)
    const int64_t bytes = nvalid * ld * 2;
    rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)p, 0, (int)(bytes < 0x7fffffff ? bytes : 0x7fffffff), 0x00020000);
    const int r = lane >> 3, pc = lane & 7;
    voff[0] = (int)(r * ld * 2) + ((pc ^ r) << 4);  // swz(8g + r) = r ^ (g & 1)
    voff[1] = (int)(r * ld * 2) + ((pc ^ r ^ 1) << 4);
    step = (int)(8 * ld * 2);
  }
  // DMA instructions LO .. HI-1 of wave slot `slot` (0..7): instruction i carries rows
  // (slot * 4 + i) * 8 .. + 7 at K offset k0 into the operand stage at `stage`.
  template <int LO, int HI>
  __device__ __forceinline__ void issue(char* stage, int slot, int k0) const {
#pragma unroll
    for (int i = LO; i < HI; ++i) {
      const int g = slot * 4 + i;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lds_ptr_t)(stage + g * 1024), 16, voff[i & 1],
                                               g * step + k0 * 2, 0, 0);
    }
  }
};

// What gemm_tile_run_8 needs of its loaders (see TileLoaders), for waves 0..3: both operands, own slot and
// the slot of wave + 4.
struct PlainTileLoaders {
  PanelLoader lp, lq;
  int k_begin, k_end;
  __device__ __forceinline__ void init(const void* P, int64_t ldp, int64_t prow0, int64_t prows, const void* Q,
                                       int64_t ldq, int64_t qrow0, int64_t qrows, int kb, int ke) {
    const int lane = threadIdx.x & 63;
    lp.init(P, ldp, prow0, prows, lane);
    lq.init(Q, ldq, qrow0, qrows, lane);
    k_begin = kb;
    k_end = ke;
  }
  template <int LO, int HI, int TAG>
  __device__ __forceinline__ void issue(char* stage, int wave, int k0) const {
    lp.issue<LO, HI>(stage, wave, k0);
    lq.issue<LO, HI>(stage + OPER_STAGE_BYTES, wave, k0);
    lp.issue<LO, HI>(stage, wave + 4, k0);
    lq.issue<LO, HI>(stage + OPER_STAGE_BYTES, wave + 4, k0);
  }
  static constexpr int DMA_PER_INDEX = 4;
  // First K stage into LDS stage 0.  No wave of the work-group may still be reading stage 0 (true at
  // kernel start and after gemm_tile_run_plain8 returns).
  __device__ __forceinline__ void issue_first(char* smem) const {
    if (plain8_leader()) issue_first_leader(smem);
  }
  // The same for a caller that is already inside its leaders' branch.
  __device__ __forceinline__ void issue_first_leader(char* smem) const {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    issue<0, 4, 0>(smem, wave, k_begin);
  }
};
// The same interface for waves 4..7: nothing to issue.
struct NoLoaders {
  int k_begin, k_end;
  template <int LO, int HI, int TAG>
  __device__ __forceinline__ void issue(char*, int, int) const {}
  static constexpr int DMA_PER_INDEX = 0;
};

// acc += P tile x Q tile^T over the K range of L (L.issue_first(smem) called by every wave; smem:
// GEMM_LDS_BYTES, 1 KiB aligned).  Accumulator layout and ALL_EARLY as gemm_tile_run<2>.  A kernel that
// runs several K ranges into one accumulator puts ONE such branch around all of them (accumulators that
// are written in a branch inside a loop get copied at every join).
template <bool ALL_EARLY>
__device__ __forceinline__ void gemm_tile_run_plain8(TileAcc<2>& acc, char* smem, const PlainTileLoaders& L) {
  if (plain8_leader()) {
    gemm_tile_run<2, 2, ALL_EARLY>(acc, smem, L);
  } else {
    NoLoaders none{L.k_begin, L.k_end};
    gemm_tile_run<2, 2, ALL_EARLY>(acc, smem, none);
  }
}

}  // namespace artk
