// Helpers shared by the LoRA linear and the MoE expert-LoRA kernels.
#pragma once
#include "common.hpp"

namespace artk {

// dst [n][R1,C1] bf16 = zero-padded copy of src [n][R0,C0] (or of each matrix's
// transpose).  One thread per destination element.
__global__ __launch_bounds__(256) static void pad_copy_bf16_kernel(const uint16_t* __restrict__ src,
                                                                   int64_t n, int64_t R0, int64_t C0,
                                                                   int transpose,
                                                                   uint16_t* __restrict__ dst,
                                                                   int64_t R1, int64_t C1) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n * R1 * C1) return;
  const int64_t b = i / (R1 * C1);
  const int64_t j = i - b * R1 * C1;
  const int64_t r = j / C1, c = j - r * C1;
  const uint16_t* sp = src + b * R0 * C0;
  uint16_t v = 0;
  if (!transpose) {
    if (r < R0 && c < C0) v = sp[r * C0 + c];
  } else {
    if (c < R0 && r < C0) v = sp[c * C0 + r];
  }
  dst[i] = v;
}

static inline int round16(int r) { return (r + 15) / 16 * 16; }

static inline int32_t launch_pad(const void* src, int64_t n, int64_t R0, int64_t C0, int transpose,
                                 uint16_t* dst, int64_t R1, int64_t C1, hipStream_t st) {
  const int64_t total = n * R1 * C1;
  pad_copy_bf16_kernel<<<(unsigned)((total + 255) / 256), 256, 0, st>>>((const uint16_t*)src, n, R0, C0,
                                                                        transpose, dst, R1, C1);
  ARTK_CHECK_LAUNCH();
  return ARTK_OK;
}

}  // namespace artk
