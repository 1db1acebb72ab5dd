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

int32_t artk_stream_copy(const void* src, void* dst, int64_t bytes, artk_stream_t stream) {
  ARTK_CHECK_ARG(src && dst, "null pointer argument");
  ARTK_CHECK_ARG(aligned16(src) && aligned16(dst) && bytes > 0 && bytes % 16 == 0,
                 "src, dst 16-byte aligned; bytes a positive multiple of 16");
  stream_copy_kernel<<<4096, 256, 0, (hipStream_t)stream>>>((const uint4*)src, (uint4*)dst, bytes / 16);
  ARTK_CHECK_LAUNCH();
  return ARTK_OK;
}

}  // extern "C"
