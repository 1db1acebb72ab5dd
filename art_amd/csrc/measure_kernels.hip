// Measurement aids of the artk library (no counterpart in the reference):
// a loop of MFMA instructions alone, which gives the bf16 rate the part sustains
// under its power limit when nothing but the matrix pipes is busy, and a plain
// streaming copy, which gives the matching figure for HBM.
#include "common.hpp"
#include "gemm_nt.hpp"
#include "gemm_4x16.hpp"
#include "gemm_half.hpp"
#include "gemm_plain8.hpp"

namespace artk {

// Every wave keeps the register tile of the GEMM main loop (4 x 2 MFMA 32x32x16
// tiles, 128 accumulators) and runs `iters` rounds of its 8 MFMAs per K = 16 step
// on operand fragments loaded once from `operands` (so the data toggles like
// real inputs), 8 waves per work-group, one work-group per CU.
__global__ __launch_bounds__(512) void mfma_loop_kernel(const uint16_t* __restrict__ operands,
                                                        int64_t n_operands, int64_t iters,
                                                        float* __restrict__ sink) {
  const int64_t gid = (int64_t)blockIdx.x * 512 + threadIdx.x;
  Frags<2> f[4];  // the four K = 16 steps of one 64-wide K stage
#pragma unroll
  for (int s = 0; s < 4; ++s) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      f[s].p[i] = *(const bf16x8*)(operands + ((gid * 24 + s * 6 + i) * 8) % (n_operands - 8));
#pragma unroll
    for (int i = 0; i < 2; ++i)
      f[s].q[i] = *(const bf16x8*)(operands + ((gid * 24 + s * 6 + 4 + i) * 8) % (n_operands - 8));
  }
  TileAcc<2> acc;
  acc.zero();
  for (int64_t it = 0; it < iters; ++it) {
#pragma unroll
    for (int s = 0; s < 4; ++s) mma_frags(acc, f[s]);
  }
  float s = 0.f;
#pragma unroll
  for (int mi = 0; mi < 4; ++mi)
#pragma unroll
    for (int ni = 0; ni < 2; ++ni)
#pragma unroll
      for (int j = 0; j < 16; ++j) s += acc.c[mi][ni][j];
  sink[gid] = s;
}

// The same amount of matrix work per round on MFMA 16x16x32 (8 x 4 tiles of 16 x 16 per
// wave, the same 128 accumulators): this shape moves a quarter of the accumulator data
// per instruction for half the flops, and sustains a higher rate under the power limit.
__global__ __launch_bounds__(512) void mfma_loop16_kernel(const uint16_t* __restrict__ operands,
                                                          int64_t n_operands, int64_t iters,
                                                          float* __restrict__ sink) {
  const int64_t gid = (int64_t)blockIdx.x * 512 + threadIdx.x;
  bf16x8 a[2][8], b[2][4];  // the two K = 32 steps of one 64-wide K stage
#pragma unroll
  for (int s = 0; s < 2; ++s) {
#pragma unroll
    for (int i = 0; i < 8; ++i) a[s][i] = *(const bf16x8*)(operands + ((gid * 24 + s * 12 + i) * 8) % (n_operands - 8));
#pragma unroll
    for (int i = 0; i < 4; ++i)
      b[s][i] = *(const bf16x8*)(operands + ((gid * 24 + s * 12 + 8 + i) * 8) % (n_operands - 8));
  }
  floatx4 c[8][4];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int e = 0; e < 4; ++e) c[i][j][e] = 0.f;
  for (int64_t it = 0; it < iters; ++it) {
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          c[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[s][i], b[s][j], c[i][j], 0, 0, 0);
  }
  float t = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int e = 0; e < 4; ++e) t += c[i][j][e];
  sink[gid] = t;
}

// LDS bandwidth probe.  Every wave of a work-group issues `iters` rounds of 16 LDS reads and
// nothing else that could limit them (the results are never consumed by a vector instruction);
// optionally one 1 KiB DMA write into another part of LDS (buffer_load ... lds from a 64 KiB
// source that stays in L2) rides along per RPD reads, the mix of the GEMM main loop (2 reads per
// DMA instruction in its 4-wave shape, 3 in its 8-wave shape).
//   KIND 0: ds_read_b128, a wave instruction reads 1 KiB contiguous
//   KIND 1: ds_read_b128 in the GEMM's fragment pattern: lane l reads the 16-byte chunk
//           ((l / 32) ^ swz(l % 32)) of row l % 32 of a tile with 128-byte rows
//   KIND 2: ds_read_b64_tr_b16 (the transposed read), 512 bytes contiguous per wave instruction
// Work-group b writes the core-clock cycles and the constant-rate (100 MHz) ticks between the
// barrier in front of the loop and the one behind it (so the slowest wave counts) to
// cycles[2b], cycles[2b + 1].
template <int NT, int KIND, int RPD>
__global__ __launch_bounds__(NT) void lds_probe_kernel(const void* __restrict__ src, int64_t iters,
                                                       int64_t* __restrict__ cycles) {
  __shared__ __attribute__((aligned(1024))) char smem[GEMM_LDS_BYTES];
  for (int i = threadIdx.x; i < GEMM_LDS_BYTES / 4; i += NT) ((int*)smem)[i] = i;
  __syncthreads();
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  int lane_off;
  if (KIND == 0) lane_off = lane * 16;
  else if (KIND == 1) lane_off = (lane & 31) * 128 + (((lane >> 5) ^ swz(lane & 31)) << 4);
  else lane_off = lane * 8;
  // reads: 16 fragments 4 KiB apart starting at this wave's 4 KiB slot (within the first 96 KiB);
  // DMA writes: four 1 KiB slots per wave in the last 32 KiB
  const uint32_t rd = lds_addr_of(smem) + (uint32_t)(wave * 4096 + lane_off);
  const uint32_t wr = lds_addr_of(smem) + 96 * 1024 + (uint32_t)wave * 4096;
  const dma_rsrc_t rsrc = dma_make_rsrc(src, 65536);
  const int voff = lane * 16;
  typedef __attribute__((__vector_size__(4 * sizeof(int)))) int intx4;
  typedef __attribute__((__vector_size__(2 * sizeof(int)))) int intx2;
  intx4 v4[4];
  intx2 v2[4];
  __syncthreads();
  const long long c0 = clock64(), w0 = wall_clock64();
  for (int64_t it = 0; it < iters; ++it) {
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      if (KIND == 2)
        asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(v2[j & 3]) : "v"(rd), "n"(j * 4096) : "memory");
      else
        asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v4[j & 3]) : "v"(rd), "n"(j * 4096) : "memory");
      if (RPD > 0 && j % RPD == RPD - 1)
        dma_load16(rsrc, voff, (int)(((it * 16 + j) & 63) * 1024), wr + (uint32_t)(j & 3) * 1024);
      if (j == 7) asm volatile("s_waitcnt lgkmcnt(8)" ::: "memory");
    }
    asm volatile("s_waitcnt lgkmcnt(8)" ::: "memory");
    if (RPD > 0) asm volatile("s_waitcnt vmcnt(24)" ::: "memory");
  }
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
  __syncthreads();  // the clock is read when the slowest wave is done
  const long long c1 = clock64(), w1 = wall_clock64();
  if (KIND == 2) asm volatile("" ::"v"(v2[0]), "v"(v2[1]), "v"(v2[2]), "v"(v2[3]));
  else asm volatile("" ::"v"(v4[0]), "v"(v4[1]), "v"(v4[2]), "v"(v4[3]));
  if (threadIdx.x == 0) {
    cycles[2 * blockIdx.x] = c1 - c0;
    cycles[2 * blockIdx.x + 1] = w1 - w0;
  }
}

template <int NT, int KIND>
static void launch_lds_probe(int rpd, unsigned blocks, hipStream_t st, const void* src, int64_t iters,
                             int64_t* cycles) {
  if (rpd == 0) lds_probe_kernel<NT, KIND, 0><<<blocks, NT, 0, st>>>(src, iters, cycles);
  else if (rpd == 2) lds_probe_kernel<NT, KIND, 2><<<blocks, NT, 0, st>>>(src, iters, cycles);
  else lds_probe_kernel<NT, KIND, 3><<<blocks, NT, 0, st>>>(src, iters, cycles);
}

// Persistent plain GEMM out[n, m] = sum_k Q[n,k] P[m,k] (bf16 out, full tiles only) on a choice of
// main loop, tile order and ablation switches: what each part of the loop costs on the hardware.
//   LOOP 0: the library's 8-wave loop (MFMA 32x32x16), 1: its pinned 4-wave loop (32x32x16),
//        2: the 4-wave loop on MFMA 16x16x32 of gemm_4x16.hpp, with the switches ABL,
//        3: the 8-wave shape on MFMA 16x16x32 (gemm_4x16.hpp), 4: 256 x 128 tiles, two work-groups per CU
//           (gemm_half.hpp)
// same_tile: every work-group fetches the tiles (b % 8, b % 8) whatever tile it computes, so all
// fetches hit in L2 (results are then wrong); group: row-operand tiles per column-operand tile of
// the tile order.  Work-group b reports its core-clock cycles and 100 MHz ticks to cycles[2b..].
struct LoopProbeParams {
  const void* P;
  const void* Q;
  uint16_t* out;
  int64_t M, N, K;
  int MT, NT, group, same_tile;
  int64_t* cycles;
};

template <int LOOP, int ABL>
__global__ __launch_bounds__(LOOP == 0 || LOOP == 3 || LOOP == 5 ? 512 : 256, LOOP == 4 ? 2 : 1) void loop_probe_kernel(
    LoopProbeParams p) {
  constexpr int NI = LOOP == 0 || LOOP == 3 || LOOP == 5 ? 2 : 4;
  __shared__ __attribute__((aligned(1024))) char smem[LOOP == 4 ? HALF_LDS_BYTES : GEMM_LDS_BYTES];
  const long long c0 = clock64(), w0 = wall_clock64();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if constexpr (LOOP == 4) {
    // 256 x 128 tiles, two work-groups per CU
    const int NT2 = p.NT * 2, n_tiles2 = p.MT * NT2;
    int t = blockIdx.x, mt, nt;
    tile_coords(xcd_remap(t, n_tiles2), p.MT, NT2, mt, nt, p.group);
    auto init = [&](HalfLoaders& L, int mt_, int nt_) {
      const int fm = p.same_tile ? (int)(blockIdx.x & 7) : mt_, fn = p.same_tile ? (int)(blockIdx.x & 7) : nt_;
      L.init(p.P, p.K, (int64_t)fm * TILE, p.M, p.Q, p.K, (int64_t)fn * HALF_Q, p.N, 0, (int)p.K);
    };
    {
      HalfLoaders first;
      init(first, mt, nt);
      first.issue_first(smem);
    }
    for (;;) {
      const int t2 = t + gridDim.x;
      const bool more = t2 < n_tiles2;
      int mt2 = 0, nt2 = 0;
      if (more) tile_coords(xcd_remap(t2, n_tiles2), p.MT, NT2, mt2, nt2, p.group);
      TileAcc<2> acc;
      acc.zero();
      {
        HalfLoaders cur;
        init(cur, mt, nt);
        gemm_half_run(acc, smem, cur);
      }
      if (more) {
        HalfLoaders nx;
        init(nx, mt2, nt2);
        nx.issue_first(smem);
      }
      const int wm = wave >> 1, wn = wave & 1;
#pragma unroll
      for (int ni = 0; ni < 2; ++ni) {
        const int64_t col = (int64_t)nt * HALF_Q + wn * 64 + ni * 32 + (lane & 31);
#pragma unroll
        for (int mi = 0; mi < 4; ++mi)
          store_block_bf16(p.out + col * p.M + (int64_t)mt * TILE + wm * 128 + mi * 32, acc.c[mi][ni], lane >> 5);
      }
      if (!more) break;
      t = t2;
      mt = mt2;
      nt = nt2;
    }
    if (threadIdx.x == 0 && p.cycles != nullptr && blockIdx.x < gridDim.x / 2) {
      p.cycles[2 * blockIdx.x] = clock64() - c0;
      p.cycles[2 * blockIdx.x + 1] = wall_clock64() - w0;
    }
    return;
  }
  if constexpr (LOOP == 5) {
    // the 8-wave loop of gemm_plain8.hpp; ABL = 1: the whole fill of a stage right after the barrier
    const int n_tiles = p.MT * p.NT;
    int t = blockIdx.x, mt, nt;
    tile_coords(xcd_remap(t, n_tiles), p.MT, p.NT, mt, nt, p.group);
    auto init = [&](PlainTileLoaders& L, int mt_, int nt_) {
      const int fm = p.same_tile ? (int)(blockIdx.x & 7) : mt_, fn = p.same_tile ? (int)(blockIdx.x & 7) : nt_;
      L.init(p.P, p.K, (int64_t)fm * TILE, p.M, p.Q, p.K, (int64_t)fn * TILE, p.N, 0, (int)p.K);
    };
    {
      PlainTileLoaders first;
      init(first, mt, nt);
      first.issue_first(smem);
    }
    for (;;) {
      const int t2 = t + gridDim.x;
      const bool more = t2 < n_tiles;
      int mt2 = 0, nt2 = 0;
      if (more) tile_coords(xcd_remap(t2, n_tiles), p.MT, p.NT, mt2, nt2, p.group);
      TileAcc<2> acc;
      acc.zero();
      {
        PlainTileLoaders cur;
        init(cur, mt, nt);
        gemm_tile_run_plain8<ABL != 0>(acc, smem, cur);
      }
      if (more) {
        PlainTileLoaders nx;
        init(nx, mt2, nt2);
        nx.issue_first(smem);
      }
      const int wm = wave_m<2>(wave), wn = wave_n<2>(wave);
#pragma unroll
      for (int ni = 0; ni < 2; ++ni) {
        const int64_t col = (int64_t)nt * TILE + acc_col<2>(wn, ni, lane);
#pragma unroll
        for (int mi = 0; mi < 4; ++mi)
          store_block_bf16(p.out + col * p.M + (int64_t)mt * TILE + wm * 128 + mi * 32, acc.c[mi][ni], lane >> 5);
      }
      if (!more) break;
      t = t2;
      mt = mt2;
      nt = nt2;
    }
    if (threadIdx.x == 0 && p.cycles != nullptr) {
      p.cycles[2 * blockIdx.x] = clock64() - c0;
      p.cycles[2 * blockIdx.x + 1] = wall_clock64() - w0;
    }
    return;
  }
  const int n_tiles = p.MT * p.NT;
  int t = blockIdx.x, mt, nt;
  tile_coords(xcd_remap(t, n_tiles), p.MT, p.NT, mt, nt, p.group);
  auto init = [&](TileLoaders<NI>& L, int mt_, int nt_) {
    const int fm = p.same_tile ? (int)(blockIdx.x & 7) : mt_, fn = p.same_tile ? (int)(blockIdx.x & 7) : nt_;
    L.init(p.P, p.K, (int64_t)fm * TILE, p.M, p.Q, p.K, (int64_t)fn * TILE, p.N, 0, (int)p.K);
  };
  {
    TileLoaders<NI> first;
    init(first, mt, nt);
    first.issue_first(smem);
  }
  for (;;) {
    const int t2 = t + gridDim.x;
    const bool more = t2 < n_tiles;
    int mt2 = 0, nt2 = 0;
    if (more) tile_coords(xcd_remap(t2, n_tiles), p.MT, p.NT, mt2, nt2, p.group);
    TileLoaders<NI> cur;
    init(cur, mt, nt);
    if constexpr (LOOP == 2) {
      TileAcc16 acc;
      acc.zero();
      gemm_tile_run_4x16<ABL>(acc, smem, cur);
      if (more) {
        TileLoaders<NI> nx;
        init(nx, mt2, nt2);
        nx.issue_first(smem);
      }
      const int wm = wave >> 1, wn = wave & 1;
#pragma unroll
      for (int nj = 0; nj < 8; ++nj) {
        const int64_t col = (int64_t)nt * TILE + wn * 128 + nj * 16 + (lane & 15);
#pragma unroll
        for (int mi = 0; mi < 8; ++mi) {
          const int64_t m = (int64_t)mt * TILE + wm * 128 + mi * 16 + (lane >> 4) * 4;
          bf16x4 o;
#pragma unroll
          for (int e = 0; e < 4; ++e) o[e] = (__bf16)acc.c[mi][nj][e];
          *(bf16x4*)(p.out + col * p.M + m) = o;
        }
      }
    } else if constexpr (LOOP == 3) {
      TileAcc16x8 acc;
      acc.zero();
      gemm_tile_run_8x16<ABL>(acc, smem, cur);
      if (more) {
        TileLoaders<NI> nx;
        init(nx, mt2, nt2);
        nx.issue_first(smem);
      }
      const int wm = wave >> 2, wn = wave & 3;
#pragma unroll
      for (int nj = 0; nj < 4; ++nj) {
        const int64_t col = (int64_t)nt * TILE + wn * 64 + nj * 16 + (lane & 15);
#pragma unroll
        for (int mi = 0; mi < 8; ++mi) {
          const int64_t m = (int64_t)mt * TILE + wm * 128 + mi * 16 + (lane >> 4) * 4;
          bf16x4 o;
#pragma unroll
          for (int e = 0; e < 4; ++e) o[e] = (__bf16)acc.c[mi][nj][e];
          *(bf16x4*)(p.out + col * p.M + m) = o;
        }
      }
    } else if constexpr (LOOP != 4) {
      TileAcc<NI> acc;
      acc.zero();
      gemm_tile_run(acc, smem, cur);
      if (more) {
        TileLoaders<NI> nx;
        init(nx, mt2, nt2);
        nx.issue_first(smem);
      }
      const int wm = wave_m<NI>(wave), wn = wave_n<NI>(wave);
#pragma unroll
      for (int ni = 0; ni < NI; ++ni) {
        const int64_t col = (int64_t)nt * TILE + acc_col<NI>(wn, ni, lane);
#pragma unroll
        for (int mi = 0; mi < 4; ++mi)
          store_block_bf16(p.out + col * p.M + (int64_t)mt * TILE + wm * 128 + mi * 32, acc.c[mi][ni], lane >> 5);
      }
    }
    if (!more) break;
    t = t2;
    mt = mt2;
    nt = nt2;
  }
  if (threadIdx.x == 0 && p.cycles != nullptr) {
    p.cycles[2 * blockIdx.x] = clock64() - c0;
    p.cycles[2 * blockIdx.x + 1] = wall_clock64() - w0;
  }
}

template <int ABL>
static void launch_loop_probe_4x16(const LoopProbeParams& p, unsigned grid, hipStream_t st) {
  loop_probe_kernel<2, ABL><<<grid, 256, 0, st>>>(p);
}

__global__ __launch_bounds__(256) void stream_copy_kernel(const uint4* __restrict__ src,
                                                          uint4* __restrict__ dst, int64_t n16) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += (int64_t)gridDim.x * 256)
    dst[i] = src[i];
}

}  // namespace artk

using namespace artk;

extern "C" {

int32_t artk_mfma_loop(const void* operands, int64_t n_operands, int64_t iters, int32_t blocks,
                       float* sink, artk_stream_t stream) {
  ARTK_CHECK_ARG(operands && sink, "null pointer argument");
  ARTK_CHECK_ARG(aligned16(operands), "operands must be 16-byte aligned");
  ARTK_CHECK_ARG(n_operands >= 4096 && n_operands % 8 == 0, "n_operands must be a multiple of 8, at least 4096");
  ARTK_CHECK_ARG(iters > 0 && blocks > 0 && blocks <= 65536, "iters and blocks must be positive (blocks <= 65536)");
  mfma_loop_kernel<<<(unsigned)blocks, 512, 0, (hipStream_t)stream>>>((const uint16_t*)operands, n_operands,
                                                                      iters, sink);
  ARTK_CHECK_LAUNCH();
  return ARTK_OK;
}

int32_t artk_mfma_loop16(const void* operands, int64_t n_operands, int64_t iters, int32_t blocks,
                         float* sink, artk_stream_t stream) {
  ARTK_CHECK_ARG(operands && sink, "null pointer argument");
  ARTK_CHECK_ARG(aligned16(operands), "operands must be 16-byte aligned");
  ARTK_CHECK_ARG(n_operands >= 4096 && n_operands % 8 == 0, "n_operands must be a multiple of 8, at least 4096");
  ARTK_CHECK_ARG(iters > 0 && blocks > 0 && blocks <= 65536, "iters and blocks must be positive (blocks <= 65536)");
  mfma_loop16_kernel<<<(unsigned)blocks, 512, 0, (hipStream_t)stream>>>((const uint16_t*)operands, n_operands,
                                                                        iters, sink);
  ARTK_CHECK_LAUNCH();
  return ARTK_OK;
}

int32_t artk_lds_probe(int32_t waves, int32_t kind, int32_t reads_per_dma, const void* src, int64_t iters,
                       int32_t blocks, int64_t* cycles, artk_stream_t stream) {
  ARTK_CHECK_ARG(src && cycles, "null pointer argument");
  ARTK_CHECK_ARG(aligned16(src), "src must be 16-byte aligned (64 KiB)");
  ARTK_CHECK_ARG(waves == 4 || waves == 8, "waves must be 4 or 8");
  ARTK_CHECK_ARG(kind >= 0 && kind <= 2, "kind must be 0 (b128 contiguous), 1 (b128 fragment pattern) or 2 (b64 transposed)");
  ARTK_CHECK_ARG(reads_per_dma == 0 || reads_per_dma == 2 || reads_per_dma == 3, "reads_per_dma must be 0, 2 or 3");
  ARTK_CHECK_ARG(iters > 0 && blocks > 0 && blocks <= 65536, "iters and blocks must be positive (blocks <= 65536)");
  hipStream_t st = (hipStream_t)stream;
  const unsigned nb = (unsigned)blocks;
  if (waves == 4) {
    if (kind == 0) launch_lds_probe<256, 0>(reads_per_dma, nb, st, src, iters, cycles);
    else if (kind == 1) launch_lds_probe<256, 1>(reads_per_dma, nb, st, src, iters, cycles);
    else launch_lds_probe<256, 2>(reads_per_dma, nb, st, src, iters, cycles);
  } else {
    if (kind == 0) launch_lds_probe<512, 0>(reads_per_dma, nb, st, src, iters, cycles);
    else if (kind == 1) launch_lds_probe<512, 1>(reads_per_dma, nb, st, src, iters, cycles);
    else launch_lds_probe<512, 2>(reads_per_dma, nb, st, src, iters, cycles);
  }
  ARTK_CHECK_LAUNCH();
  return ARTK_OK;
}

int32_t artk_gemm_loop_probe(const void* P, const void* Q, void* out, int64_t M, int64_t N, int64_t K,
                             int32_t loop, int32_t ablate, int32_t group, int32_t same_tile, int64_t* cycles,
                             artk_stream_t stream) {
  ARTK_CHECK_ARG(P && Q && out, "null pointer argument");
  ARTK_CHECK_ARG(aligned16(P) && aligned16(Q) && aligned16(out), "pointers must be 16-byte aligned");
  ARTK_CHECK_ARG(M >= 2048 && N >= 2048 && K >= 128 && M % 256 == 0 && N % 256 == 0 && K % 64 == 0,
                 "M and N must be multiples of 256 (at least 2048), K a multiple of 64 (at least 128)");
  ARTK_CHECK_ARG(loop >= 0 && loop <= 5,
                 "loop must be 0 (8-wave), 1 (4-wave 32x32x16), 2 (4-wave 16x16x32), 3 (8-wave 16x16x32), 4 "
                 "(256 x 128 tiles, two work-groups per CU) or 5 (8-wave, DMA issued by the first wave of each SIMD)");
  ARTK_CHECK_ARG(ablate >= 0 && ablate <= 7 && ablate != 6 &&
                     (ablate == 0 || loop == 2 || (loop == 3 && ablate != 3) || (loop == 5 && ablate == 1)),
                 "ablate: bits 1 (no DMA), 2 (no barrier), 4 (no LDS reads); 6 is not built (nor 3 with loop 3); only "
                 "with loops 2 and 3; with loop 5, 1 selects the whole fill right after the barrier");
  ARTK_CHECK_ARG(group >= 1 && group <= 64, "group must be in 1..64");
  LoopProbeParams p;
  p.P = P;
  p.Q = Q;
  p.out = (uint16_t*)out;
  p.M = M;
  p.N = N;
  p.K = K;
  p.MT = (int)(M / TILE);
  p.NT = (int)(N / TILE);
  p.group = group;
  p.same_tile = same_tile != 0;
  p.cycles = cycles;
  int cus = 0, dev = 0;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
    cus = 256;
  const int64_t tiles = (int64_t)p.MT * p.NT;
  const unsigned grid = (unsigned)(tiles < cus ? tiles : cus);
  hipStream_t st = (hipStream_t)stream;
  if (loop == 0) loop_probe_kernel<0, 0><<<grid, 512, 0, st>>>(p);
  else if (loop == 1) loop_probe_kernel<1, 0><<<grid, 256, 0, st>>>(p);
  else if (loop == 3) {
    switch (ablate) {
      case 0: loop_probe_kernel<3, 0><<<grid, 512, 0, st>>>(p); break;
      case 1: loop_probe_kernel<3, 1><<<grid, 512, 0, st>>>(p); break;
      case 2: loop_probe_kernel<3, 2><<<grid, 512, 0, st>>>(p); break;
      case 4: loop_probe_kernel<3, 4><<<grid, 512, 0, st>>>(p); break;
      case 5: loop_probe_kernel<3, 5><<<grid, 512, 0, st>>>(p); break;
      default: loop_probe_kernel<3, 7><<<grid, 512, 0, st>>>(p); break;
    }
  }
  else if (loop == 5) {
    if (ablate == 0) loop_probe_kernel<5, 0><<<grid, 512, 0, st>>>(p);
    else loop_probe_kernel<5, 1><<<grid, 512, 0, st>>>(p);
  }
  else if (loop == 4) {
    const int64_t tiles2 = tiles * 2;
    loop_probe_kernel<4, 0><<<(unsigned)(tiles2 < 2 * cus ? tiles2 : 2 * cus), 256, 0, st>>>(p);
  }
  else switch (ablate) {
    case 0: launch_loop_probe_4x16<0>(p, grid, st); break;
    case 1: launch_loop_probe_4x16<1>(p, grid, st); break;
    case 2: launch_loop_probe_4x16<2>(p, grid, st); break;
    case 3: launch_loop_probe_4x16<3>(p, grid, st); break;
    case 4: launch_loop_probe_4x16<4>(p, grid, st); break;
    case 5: launch_loop_probe_4x16<5>(p, grid, st); break;
    default: launch_loop_probe_4x16<7>(p, grid, st); break;
  }
  ARTK_CHECK_LAUNCH();
  return ARTK_OK;
}

int32_t artk_stream_copy(const void* src, void* dst, int64_t bytes, artk_stream_t stream) {
  ARTK_CHECK_ARG(src && dst, "null pointer argument");
  ARTK_CHECK_ARG(aligned16(src) && aligned16(dst) && bytes > 0 && bytes % 16 == 0,
                 "src, dst 16-byte aligned; bytes a positive multiple of 16");
  stream_copy_kernel<<<4096, 256, 0, (hipStream_t)stream>>>((const uint4*)src, (uint4*)dst, bytes / 16);
  ARTK_CHECK_LAUNCH();
  return ARTK_OK;
}

}  // extern "C"
