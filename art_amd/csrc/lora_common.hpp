// Helpers shared by the LoRA linear and the MoE expert-LoRA kernels: the rank-r
// extra K steps of the GEMM epilogue and the skinny products.
#pragma once
#include "common.hpp"
#include "gemm_nt.hpp"

namespace artk {

static inline int round16(int r) { return (r + 15) / 16 * 16; }

// acc += sum_e Qe[col, e] * Pe[row, e] for e < rp (rp a multiple of 16), as extra
// K = 16 MFMA steps.  The operand fragments come straight from global memory in
// MFMA layout: 16 bytes per lane = 8 consecutive e of row (lane % 32), first or
// second half of the step by lane / 32.  Chunks at or past *_valid read as zero,
// so a [rows, r] factor with r % 8 == 0 needs no padded copy.
template <int NI>
__device__ __forceinline__ void lowrank_steps(TileAcc<NI>& acc, const uint16_t* Pe, int pe_ld, int pe_valid,
                                              const int64_t (&prow)[4], const uint16_t* Qe, int qe_ld,
                                              int qe_valid, const int64_t (&qrow)[NI], int rp) {
  const int half = (threadIdx.x & 63) >> 5;
  for (int e0 = 0; e0 < rp; e0 += 16) {
    const int e = e0 + half * 8;
    // Every lane loads (a chunk past the end reads chunk 0 instead and is zeroed
    // afterwards): loads under a lane mask would each be waited for in turn.
    const bool p_ok = e < pe_valid, q_ok = e < qe_valid;
    const int ep = p_ok ? e : 0, eq = q_ok ? e : 0;
    Frags<NI> f;
    const bf16x8 z = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < 4; ++i) f.p[i] = *(const bf16x8*)(Pe + prow[i] * pe_ld + ep);
#pragma unroll
    for (int i = 0; i < NI; ++i) f.q[i] = *(const bf16x8*)(Qe + qrow[i] * qe_ld + eq);
#pragma unroll
    for (int i = 0; i < 4; ++i) f.p[i] = p_ok ? f.p[i] : z;
#pragma unroll
    for (int i = 0; i < NI; ++i) f.q[i] = q_ok ? f.q[i] : z;
    mma_frags(acc, f);
  }
}

// Row products with MFMA 16x16x32: for the 16 rows held by the caller (lane % 16
// selects the row behind xp / the factor row behind mp, lane / 16 the 8-element
// K slice), accumulate over k = wave*32, wave*32 + 128, ...  Four independent
// accumulators keep eight 16-byte loads in flight per lane.
__device__ __forceinline__ floatx4 rowdot_accumulate(const uint16_t* xp, const uint16_t* mp,
                                                     bool m_valid, int64_t K, int wave) {
  floatx4 a0 = {0.f, 0.f, 0.f, 0.f}, a1 = a0, a2 = a0, a3 = a0;
  const bf16x8 z = {0, 0, 0, 0, 0, 0, 0, 0};
  int64_t k = (int64_t)wave * 32;
  for (; k + 384 < K; k += 512) {
    const bf16x8 x0 = *(const bf16x8*)(xp + k), x1 = *(const bf16x8*)(xp + k + 128);
    const bf16x8 x2 = *(const bf16x8*)(xp + k + 256), x3 = *(const bf16x8*)(xp + k + 384);
    const bf16x8 m0 = m_valid ? *(const bf16x8*)(mp + k) : z;
    const bf16x8 m1 = m_valid ? *(const bf16x8*)(mp + k + 128) : z;
    const bf16x8 m2 = m_valid ? *(const bf16x8*)(mp + k + 256) : z;
    const bf16x8 m3 = m_valid ? *(const bf16x8*)(mp + k + 384) : z;
    a0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(x0, m0, a0, 0, 0, 0);
    a1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(x1, m1, a1, 0, 0, 0);
    a2 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(x2, m2, a2, 0, 0, 0);
    a3 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(x3, m3, a3, 0, 0, 0);
  }
  for (; k < K; k += 128) {
    const bf16x8 x0 = *(const bf16x8*)(xp + k);
    const bf16x8 m0 = m_valid ? *(const bf16x8*)(mp + k) : z;
    a0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(x0, m0, a0, 0, 0, 0);
  }
  return (a0 + a1) + (a2 + a3);
}

// Sum the four waves' accumulators (wave 0 ends up with the total).
__device__ __forceinline__ floatx4 rowdot_block_sum(floatx4 acc, floatx4 (*red)[64]) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (wave > 0) red[wave - 1][lane] = acc;
  __syncthreads();
  if (wave == 0) {
    acc += red[0][lane];
    acc += red[1][lane];
    acc += red[2][lane];
  }
  return acc;
}

// 4 bf16 -> 4 floats.
__device__ __forceinline__ void unpack2(uint32_t w, float& lo, float& hi) {
  lo = __uint_as_float(w << 16);
  hi = __uint_as_float(w & 0xffff0000u);
}

// dst[c, r] = src[r, c] for n bf16 matrices [R, C] with R and C multiples of 8 (LoRA factors: one
// dimension is the rank); blockIdx.y selects one of two jobs so that both transposes of a LoRA
// backward share a launch.  A thread turns an 8 x 8 block in registers: eight 16-byte loads along
// the rows of src, eight 16-byte stores along the rows of dst.
struct SmallTranspose {
  const uint16_t* src;
  uint16_t* dst;
  int64_t n, R, C;  // n matrices of [R, C]
};
__device__ __forceinline__ void small_transpose_one(const SmallTranspose& t) {
  const int64_t RB = t.R / 8, CB = t.C / 8;
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= t.n * RB * CB) return;
  const int64_t m = i / (RB * CB), j = i - m * RB * CB;
  const int64_t rb = j / CB, cb = j - rb * CB;
  const uint16_t* src = t.src + m * t.R * t.C + rb * 8 * t.C + cb * 8;
  uint16_t* dst = t.dst + m * t.R * t.C + cb * 8 * t.R + rb * 8;
  uint32_t in[8][4];  // in[r][k]: columns 2k, 2k + 1 of row r
#pragma unroll
  for (int r = 0; r < 8; ++r) {
    const uint4 v = *(const uint4*)(src + r * t.C);
    in[r][0] = v.x;
    in[r][1] = v.y;
    in[r][2] = v.z;
    in[r][3] = v.w;
  }
#pragma unroll
  for (int c = 0; c < 8; ++c) {
    uint32_t o[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const uint32_t lo = (in[2 * k][c >> 1] >> (16 * (c & 1))) & 0xffffu;
      const uint32_t hi = (in[2 * k + 1][c >> 1] >> (16 * (c & 1))) & 0xffffu;
      o[k] = lo | (hi << 16);
    }
    *(uint4*)(dst + c * t.R) = make_uint4(o[0], o[1], o[2], o[3]);
  }
}
__global__ __launch_bounds__(256) static void small_transpose2_kernel(SmallTranspose a, SmallTranspose b) {
  small_transpose_one(blockIdx.y == 0 ? a : b);
}
// Up to 8 jobs in one launch (the factors of several projections).
struct SmallTransposeMulti {
  SmallTranspose t[8];
  int n;
};
__global__ __launch_bounds__(256) static void small_transpose_multi_kernel(SmallTransposeMulti m) {
  small_transpose_one(m.t[blockIdx.y]);
}
static inline int32_t launch_small_transpose_multi(const SmallTransposeMulti& m, hipStream_t st) {
  int64_t big = 0;
  for (int i = 0; i < m.n; ++i) {
    const int64_t e = m.t[i].n * m.t[i].R * m.t[i].C / 64;  // 8 x 8 blocks
    big = e > big ? e : big;
  }
  dim3 grid((unsigned)((big + 255) / 256), (unsigned)m.n);
  small_transpose_multi_kernel<<<grid, 256, 0, st>>>(m);
  ARTK_CHECK_LAUNCH();
  return ARTK_OK;
}

static inline int32_t launch_small_transpose2(const void* s0, void* d0, int64_t n0, int64_t R0, int64_t C0,
                                              const void* s1, void* d1, int64_t n1, int64_t R1, int64_t C1,
                                              hipStream_t st) {
  SmallTranspose a{(const uint16_t*)s0, (uint16_t*)d0, n0, R0, C0};
  SmallTranspose b{(const uint16_t*)s1, (uint16_t*)d1, n1, R1, C1};
  const int64_t big = (n0 * R0 * C0 > n1 * R1 * C1 ? n0 * R0 * C0 : n1 * R1 * C1) / 64;  // 8 x 8 blocks
  dim3 grid((unsigned)((big + 255) / 256), 2);
  small_transpose2_kernel<<<grid, 256, 0, st>>>(a, b);
  ARTK_CHECK_LAUNCH();
  return ARTK_OK;
}

}  // namespace artk
