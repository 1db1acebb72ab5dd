// Measurement aids of the artk library (no counterpart in the reference):
// a loop of MFMA instructions alone, which gives the bf16 rate the part sustains
// under its power limit when nothing but the matrix pipes is busy, and a plain
// streaming copy, which gives the matching figure for HBM.
#include "common.hpp"
#include "gemm_nt.hpp"

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

int32_t artk_stream_copy(const void* src, void* dst, int64_t bytes, artk_stream_t stream) {
  ARTK_CHECK_ARG(src && dst, "null pointer argument");
  ARTK_CHECK_ARG(aligned16(src) && aligned16(dst) && bytes > 0 && bytes % 16 == 0,
                 "src, dst 16-byte aligned; bytes a positive multiple of 16");
  stream_copy_kernel<<<4096, 256, 0, (hipStream_t)stream>>>((const uint4*)src, (uint4*)dst, bytes / 16);
  ARTK_CHECK_LAUNCH();
  return ARTK_OK;
}

}  // extern "C"
