// 4-bit NormalFloat (NF4) base weights -> bf16, gfx950.
//
// The reference loads the base model with `load_in_4bit=True`
// (src/art/dev/model.py:29): bitsandbytes keeps each frozen linear weight as
// 4-bit NF4 codes, two per byte (first element in the high nibble), with one
// absolute maximum per block of 64 elements, optionally itself quantised to
// 8 bits ("double quantisation": a 256-entry code book, one fp32 scale per 256
// blocks, and a scalar offset).  The LoRA GEMMs of this library take bf16
// weights; this kernel produces them from the packed form.  HBM-bound:
// 0.5 B (+ 0.06 B of scales) read and 2 B written per element, a few per cent
// of the time of the GEMM that follows.
#include "common.hpp"

namespace artk {

// The 16 NF4 levels (Dettmers et al., "QLoRA", 2023, appendix E; the
// bitsandbytes code book for quant_type="nf4").
__constant__ float NF4_LEVELS[16] = {
    -1.0f, -0.6961928009986877f, -0.5250730514526367f, -0.39491748809814453f,
    -0.28444138169288635f, -0.18477343022823334f, -0.09105003625154495f, 0.0f,
    0.07958029955625534f, 0.16093020141124725f, 0.24611230194568634f, 0.33791524171829224f,
    0.44070982933044434f, 0.5626170039176941f, 0.7229568362236023f, 1.0f};

struct Nf4Params {
  const uint8_t* packed;     // n / 2 bytes
  const float* absmax;       // [n / blocksize] or nullptr
  const uint8_t* absmax_q;   // [n / blocksize] (nested form)
  const float* code2;        // [256]
  const float* absmax2;      // [ceil(n / blocksize / 256)]
  float offset;
  int64_t n;
  int blocksize;             // power of two, >= 32
  uint16_t* out;             // [n] bf16
};

// One thread: 4 packed bytes = 8 consecutive elements, so a wave reads 256
// contiguous bytes and writes 1 KiB contiguous.
__global__ __launch_bounds__(256) void nf4_dequant_kernel(Nf4Params p) {
  __shared__ float lut[4][16];   // one copy per wave to spread the bank load
  if (threadIdx.x < 64) lut[threadIdx.x >> 4][threadIdx.x & 15] = NF4_LEVELS[threadIdx.x & 15];
  __syncthreads();
  const float* t = lut[threadIdx.x >> 6];
  const int64_t stride = (int64_t)gridDim.x * 256 * 8;
  for (int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 8; i < p.n; i += stride) {
    const int64_t blk = i / p.blocksize;
    float scale;
    if (p.absmax != nullptr) {
      scale = p.absmax[blk];
    } else {
      // separate multiply and add: the CPU restatement does not contract them
      scale = __fadd_rn(__fmul_rn(p.code2[p.absmax_q[blk]], p.absmax2[blk >> 8]), p.offset);
    }
    const uint32_t w = *(const uint32_t*)(p.packed + i / 2);
    uint32_t o[4];
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const uint32_t byte = (w >> (8 * b)) & 0xff;
      const float hi = t[byte >> 4] * scale;
      const float lo = t[byte & 15] * scale;
      o[b] = (uint32_t)f32_to_bf16(hi) | ((uint32_t)f32_to_bf16(lo) << 16);
    }
    *(uint4*)(p.out + i) = make_uint4(o[0], o[1], o[2], o[3]);
  }
}

// Same values written transposed: the weight is [R, C] (C elements per row, quantisation blocks
// run along a row), the output is bf16 [C, R].  A work-group turns a 64 x 64 tile through LDS:
// 4-byte packed reads along the rows, 8-byte stores along the output rows.
__global__ __launch_bounds__(256) void nf4_dequant_t_kernel(Nf4Params p, int64_t R, int64_t C) {
  __shared__ float lut[16];
  __shared__ uint16_t tile[64][66];
  if (threadIdx.x < 16) lut[threadIdx.x] = NF4_LEVELS[threadIdx.x];
  __syncthreads();
  const int64_t r0 = (int64_t)blockIdx.y * 64, c0 = (int64_t)blockIdx.x * 64;
  // 64 rows x 8 groups of 8 elements: thread -> (row, group); two passes
  for (int i = threadIdx.x; i < 64 * 8; i += 256) {
    const int rr = i >> 3, g8 = (i & 7) * 8;
    const int64_t r = r0 + rr, c = c0 + g8;
    if (r < R && c < C) {
      const int64_t e = r * C + c;
      const int64_t blk = e / p.blocksize;
      float scale;
      if (p.absmax != nullptr)
        scale = p.absmax[blk];
      else
        scale = __fadd_rn(__fmul_rn(p.code2[p.absmax_q[blk]], p.absmax2[blk >> 8]), p.offset);
      const uint32_t w = *(const uint32_t*)(p.packed + e / 2);
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        const uint32_t byte = (w >> (8 * b)) & 0xff;
        tile[rr][g8 + 2 * b] = f32_to_bf16(lut[byte >> 4] * scale);
        tile[rr][g8 + 2 * b + 1] = f32_to_bf16(lut[byte & 15] * scale);
      }
    }
  }
  __syncthreads();
  // output rows c0 + cc, 64 consecutive r each: thread -> (cc, 4 consecutive r)
  for (int i = threadIdx.x; i < 64 * 16; i += 256) {
    const int cc = i >> 4, r4 = (i & 15) * 4;
    const int64_t c = c0 + cc, r = r0 + r4;
    if (c < C && r < R) {  // R % 8 == 0: a group of 4 is inside or outside as a whole
      const uint32_t lo = (uint32_t)tile[r4][cc] | ((uint32_t)tile[r4 + 1][cc] << 16);
      const uint32_t hi = (uint32_t)tile[r4 + 2][cc] | ((uint32_t)tile[r4 + 3][cc] << 16);
      *(uint2*)(p.out + c * R + r) = make_uint2(lo, hi);
    }
  }
}

static int32_t check_nf4(const void* packed, const float* absmax, const void* absmax_q, const float* code2,
                         const float* absmax2, int64_t n, int32_t blocksize, const void* out) {
  ARTK_CHECK_ARG(packed && out, "null pointer argument");
  ARTK_CHECK_ARG(absmax != nullptr || (absmax_q && code2 && absmax2),
                 "give absmax, or absmax_q + code2 + absmax2");
  ARTK_CHECK_ARG(aligned16(packed) && aligned16(out), "packed and out must be 16-byte aligned");
  if (n <= 0 || n % 32 != 0 || blocksize < 32 || (blocksize & (blocksize - 1)) != 0 || n % blocksize != 0) {
    set_error("n (%lld) must be a positive multiple of the block size (%d), a power of two >= 32",
              (long long)n, blocksize);
    return ARTK_ERR_UNSUPPORTED_SHAPE;
  }
  return ARTK_OK;
}

static Nf4Params nf4_params(const void* packed, const float* absmax, const void* absmax_q, const float* code2,
                            const float* absmax2, float offset, int64_t n, int32_t blocksize, void* out) {
  Nf4Params p;
  p.packed = (const uint8_t*)packed;
  p.absmax = absmax;
  p.absmax_q = (const uint8_t*)absmax_q;
  p.code2 = code2;
  p.absmax2 = absmax2;
  p.offset = offset;
  p.n = n;
  p.blocksize = blocksize;
  p.out = (uint16_t*)out;
  return p;
}

}  // namespace artk

using namespace artk;

extern "C" {

int32_t artk_nf4_dequant(const void* packed, const float* absmax, const void* absmax_q,
                         const float* code2, const float* absmax2, float offset, int64_t n,
                         int32_t blocksize, void* out_bf16, artk_stream_t stream) {
  int32_t rc = check_nf4(packed, absmax, absmax_q, code2, absmax2, n, blocksize, out_bf16);
  if (rc) return rc;
  Nf4Params p = nf4_params(packed, absmax, absmax_q, code2, absmax2, offset, n, blocksize, out_bf16);
  const int64_t blocks = (n / 8 + 255) / 256;
  nf4_dequant_kernel<<<(unsigned)(blocks < 16384 ? blocks : 16384), 256, 0, (hipStream_t)stream>>>(p);
  ARTK_CHECK_LAUNCH();
  return ARTK_OK;
}

int32_t artk_nf4_dequant_t(const void* packed, const float* absmax, const void* absmax_q,
                           const float* code2, const float* absmax2, float offset, int64_t rows,
                           int64_t cols, int32_t blocksize, void* out_bf16, artk_stream_t stream) {
  ARTK_CHECK_ARG(rows > 0 && cols > 0 && rows % 8 == 0 && cols % 8 == 0, "rows and cols must be positive multiples of 8");
  ARTK_CHECK_ARG(rows < 65536 * 64, "too many rows");
  int32_t rc = check_nf4(packed, absmax, absmax_q, code2, absmax2, rows * cols, blocksize, out_bf16);
  if (rc) return rc;
  Nf4Params p = nf4_params(packed, absmax, absmax_q, code2, absmax2, offset, rows * cols, blocksize, out_bf16);
  dim3 grid((unsigned)((cols + 63) / 64), (unsigned)((rows + 63) / 64));
  nf4_dequant_t_kernel<<<grid, 256, 0, (hipStream_t)stream>>>(p, rows, cols);
  ARTK_CHECK_LAUNCH();
  return ARTK_OK;
}

}  // extern "C"
