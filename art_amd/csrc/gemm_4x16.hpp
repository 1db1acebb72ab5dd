// Measurement variant of the NT GEMM main loop (see gemm_nt.hpp): the 4-wave work-group shape
// (2 x 2 waves, wave tile 128 x 128, one wave per SIMD) on MFMA 16x16x32 instead of 32x32x16,
// instruction order pinned, with switches that take parts of the loop away.  It exists to
// answer, on the hardware, what each part of the loop costs; the library's kernels use the
// loops of gemm_nt.hpp.
//
// Same stages, swizzle, DMA instructions and barrier as gemm_nt.hpp.  A K = 32 step is 64 MFMAs
// (8 x 8 tiles of 16 x 16) written as 16 groups of {4 MFMAs, 1 fragment read of the next step,
// at most 1 DMA instruction} with a scheduling barrier after each group.  The MFMAs are issued
// from inline assembly with the accumulator tied in place ("+a"): written with the builtin, the
// register allocator moved a sixth of the 256 accumulators between AGPRs and VGPRs in every K
// step (88 v_accvgpr moves per 128 MFMAs).  The compiler therefore does not know that these are
// MFMAs: in-place accumulation needs no software wait states, and the loop ends with explicit
// s_nop before anything reads the accumulators.
#pragma once
#include "common.hpp"
#include "gemm_nt.hpp"

namespace artk {

// Switches (bits of ABL): what is taken out of the loop.  Results are wrong with any of them set.
constexpr int ABL_NO_DMA = 1;      // no fill of the next stages (operands stay as first loaded)
constexpr int ABL_NO_BARRIER = 2;  // no wait for the fill and no work-group barrier per K step
constexpr int ABL_NO_LDS_READ = 4; // fragments are read once, before the loop

struct TileAcc16 {
  floatx4 c[8][8];  // [mi][nj]: row wm*128 + mi*16 + (lane/16)*4 + e, column wn*128 + nj*16 + lane%16
  __device__ __forceinline__ void zero() {
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j)
#pragma unroll
        for (int e = 0; e < 4; ++e) c[i][j][e] = 0.f;
  }
};
struct Frags16 {
  bf16x8 p[8], q[8];
};

// Fragment G of a step's read order p0 q0..q7 p1..p7 (what the first MFMAs need comes first).
template <int G>
__device__ __forceinline__ void read_frag16(Frags16& f, const char* sp, const char* sq, int off) {
  if constexpr (G == 0) f.p[0] = *(const bf16x8*)(sp + off);
  else if constexpr (G <= 8) f.q[G - 1] = *(const bf16x8*)(sq + off + (G - 1) * 2048);
  else f.p[G - 8] = *(const bf16x8*)(sp + off + (G - 8) * 2048);
}

// The four MFMAs of group G: row tile G / 2, column tiles 4 (G % 2) .. +3, serpentine.
template <int G>
__device__ __forceinline__ void mma_group16(TileAcc16& acc, const Frags16& f) {
  constexpr int i = G / 2;
  constexpr int jh = (i & 1) ? 1 - (G & 1) : (G & 1);
#pragma unroll
  for (int jj = 0; jj < 4; ++jj) {
    const int j = (i & 1) ? jh * 4 + 3 - jj : jh * 4 + jj;
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc.c[i][j]) : "v"(f.p[i]), "v"(f.q[j]));
  }
}

// DN: ordinal of the DMA instruction of this group among the 16 of a stage (order p0 q0 p1 q1 ...),
// -1: none.  TAG is unused (it keeps the specialisations of different steps apart).
template <int ABL, int G, int DN, int TAG>
__device__ __forceinline__ void group16(TileAcc16& acc, const Frags16& use, Frags16& fill, const char* sp,
                                        const char* sq, int off, const OperandLoader<4>& lp,
                                        const OperandLoader<4>& lq, char* dst, int wave, int k) {
  constexpr int D = DN < 0 || DN >= 16 ? -1 : (DN & 1) ? 8 + DN / 2 : DN / 2;
  mma_group16<G>(acc, use);
  if constexpr (!(ABL & ABL_NO_LDS_READ)) read_frag16<G>(fill, sp, sq, off);
  if constexpr (!(ABL & ABL_NO_DMA)) {
    if constexpr (D >= 0 && D < 8) lp.issue_one(dst, wave, k, D);
    if constexpr (D >= 8 && D < 16) lq.issue_one(dst + OPER_STAGE_BYTES, wave, k, D - 8);
  }
  __builtin_amdgcn_sched_barrier(0);
}

// One K = 32 step; DMA instructions N0 .. N0+ND-1 of the stage ride in its first groups.
template <int ABL, int N0, int ND>
__device__ __forceinline__ void step16(TileAcc16& acc, const Frags16& use, Frags16& fill, const char* sp,
                                       const char* sq, int off, const OperandLoader<4>& lp,
                                       const OperandLoader<4>& lq, char* dst, int wave, int k) {
#define ARTK_G16(G) \
  group16<ABL, G, (G < ND ? N0 + G : -1), N0 * 100 + ND>(acc, use, fill, sp, sq, off, lp, lq, dst, wave, k)
  ARTK_G16(0); ARTK_G16(1); ARTK_G16(2); ARTK_G16(3); ARTK_G16(4); ARTK_G16(5); ARTK_G16(6); ARTK_G16(7);
  ARTK_G16(8); ARTK_G16(9); ARTK_G16(10); ARTK_G16(11); ARTK_G16(12); ARTK_G16(13); ARTK_G16(14); ARTK_G16(15);
#undef ARTK_G16
}

// acc += P tile x Q tile^T over the K range of L (L.issue_first(smem) already called).  Twelve of the
// sixteen DMA instructions of stage kt + 2 are issued in the step after the barrier that frees its
// buffer, the other four at the start of the next step (all sixteen at once: 0.5 % slower; eight and
// eight: 2.5 % slower, the last ones then land too late).
template <int ABL>
__device__ __forceinline__ void gemm_tile_run_4x16(TileAcc16& acc, char* smem, const TileLoaders<4>& L) {
  constexpr int DA = 12;
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int wm = wave >> 1, wn = wave & 1;
  const OperandLoader<4>& lp = L.lp;
  const OperandLoader<4>& lq = L.lq;
  const int k_begin = L.k_begin, k_end = L.k_end;
  int off[2];  // lane l: row l % 16 of a 16-row fragment, 16-byte chunk 4 ks + l / 16, swizzled
  {
    const int rl = lane & 15;
    const int f = swz(rl);
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) off[ks] = rl * 128 + (((ks * 4 + (lane >> 4)) ^ f) << 4);
  }
  const int p_wave_off = wm * 128 * 128;
  const int q_wave_off = OPER_STAGE_BYTES + wn * 128 * 128;
  const int nk = (k_end - k_begin) / BK;
  const int k_last = k_end - BK;

  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  Frags16 fa, fb;
  {
    const char* sp = smem + p_wave_off;
    const char* sq = smem + q_wave_off;
    read_frag16<0>(fa, sp, sq, off[0]); read_frag16<1>(fa, sp, sq, off[0]); read_frag16<2>(fa, sp, sq, off[0]);
    read_frag16<3>(fa, sp, sq, off[0]); read_frag16<4>(fa, sp, sq, off[0]); read_frag16<5>(fa, sp, sq, off[0]);
    read_frag16<6>(fa, sp, sq, off[0]); read_frag16<7>(fa, sp, sq, off[0]); read_frag16<8>(fa, sp, sq, off[0]);
    read_frag16<9>(fa, sp, sq, off[0]); read_frag16<10>(fa, sp, sq, off[0]); read_frag16<11>(fa, sp, sq, off[0]);
    read_frag16<12>(fa, sp, sq, off[0]); read_frag16<13>(fa, sp, sq, off[0]); read_frag16<14>(fa, sp, sq, off[0]);
    read_frag16<15>(fa, sp, sq, off[0]);
    if constexpr ((ABL & ABL_NO_LDS_READ) != 0) fb = fa;
    if constexpr (!(ABL & ABL_NO_DMA)) {
      const int k1 = k_begin + BK < k_last ? k_begin + BK : k_last;
#pragma unroll
      for (int n = 0; n < DA; ++n) {
        const int d = (n & 1) ? 8 + n / 2 : n / 2;
        if (d < 8) lp.issue_one(smem + STAGE_BYTES, wave, k1, d);
        else lq.issue_one(smem + STAGE_BYTES + OPER_STAGE_BYTES, wave, k1, d - 8);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  }
  for (int kt = 0; kt < nk; ++kt) {
    char* cur = smem + (kt & 1) * STAGE_BYTES;
    char* nxt = smem + ((kt + 1) & 1) * STAGE_BYTES;
    const char* sp = cur + p_wave_off;
    const char* sq = cur + q_wave_off;
    int k1 = k_begin + (kt + 1) * BK;
    k1 = k1 < k_last ? k1 : k_last;
    // first half of this stage (fa); the rest of the next stage's DMA
    step16<ABL, DA, 16 - DA>(acc, fa, fb, sp, sq, off[1], lp, lq, nxt, wave, k1);
    if constexpr (!(ABL & ABL_NO_BARRIER)) {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
    }
    int k2 = k_begin + (kt + 2) * BK;
    k2 = k2 < k_last ? k2 : k_last;
    // second half (fb) while the first fragments of the next stage are read; DMA of the stage after next
    step16<ABL, 0, DA>(acc, fb, fa, nxt + p_wave_off, nxt + q_wave_off, off[0], lp, lq, cur, wave, k2);
  }
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
  __syncthreads();
  asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");  // the MFMAs above are invisible to the compiler
}

// ----------------------------------------------------------------------------
// The 8-wave work-group shape (2 x 4 waves, wave tile 128 x 64, two waves per SIMD) on MFMA
// 16x16x32: 8 x 4 tiles of 16 x 16 per wave, 128 accumulators per lane.  A K = 32 step is 32 MFMAs,
// 12 fragment reads of the next step and 4 DMA instructions; the compiler orders them under
// scheduling-group barriers as in the 8-wave loop of gemm_nt.hpp (the second wave of the SIMD
// covers what stalls remain).
struct TileAcc16x8 {
  floatx4 c[8][4];  // [mi][nj]: row wm*128 + mi*16 + (lane/16)*4 + e, column wn*64 + nj*16 + lane%16
  __device__ __forceinline__ void zero() {
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int e = 0; e < 4; ++e) c[i][j][e] = 0.f;
  }
};
struct Frags16x8 {
  bf16x8 p[8], q[4];
};
__device__ __forceinline__ void load_frags16x8(Frags16x8& f, const char* sp, const char* sq, int off) {
#pragma unroll
  for (int j = 0; j < 4; ++j) f.q[j] = *(const bf16x8*)(sq + off + j * 2048);
#pragma unroll
  for (int i = 0; i < 8; ++i) f.p[i] = *(const bf16x8*)(sp + off + i * 2048);
}
__device__ __forceinline__ void mma_frags16x8(TileAcc16x8& acc, const Frags16x8& f) {
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
      acc.c[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f.p[i], f.q[j], acc.c[i][j], 0, 0, 0);
}

template <int ABL = 0>
__device__ __forceinline__ void gemm_tile_run_8x16(TileAcc16x8& acc, char* smem, const TileLoaders<2>& L) {
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int wm = wave >> 2, wn = wave & 3;
  const OperandLoader<2>& lp = L.lp;
  const OperandLoader<2>& lq = L.lq;
  const int k_begin = L.k_begin, k_end = L.k_end;
  int off[2];
  {
    const int rl = lane & 15;
    const int f = swz(rl);
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) off[ks] = rl * 128 + (((ks * 4 + (lane >> 4)) ^ f) << 4);
  }
  const int p_wave_off = wm * 128 * 128;
  const int q_wave_off = OPER_STAGE_BYTES + wn * 64 * 128;
  const int nk = (k_end - k_begin) / BK;

  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  if (nk > 1 && !(ABL & ABL_NO_DMA)) {
    lp.template issue<0, 2, 500 + ABL>(smem + STAGE_BYTES, wave, k_begin + BK);
    lq.template issue<0, 2, 500 + ABL>(smem + STAGE_BYTES + OPER_STAGE_BYTES, wave, k_begin + BK);
  }
  Frags16x8 fa, fb;
  load_frags16x8(fa, smem + p_wave_off, smem + q_wave_off, off[0]);
  if constexpr ((ABL & ABL_NO_LDS_READ) != 0) fb = fa;

  auto k_step = [&](int kt, auto late_tag, auto ahead_tag) {
    constexpr bool LATE = decltype(late_tag)::value, AHEAD = decltype(ahead_tag)::value;
    char* cur = smem + (kt & 1) * STAGE_BYTES;
    char* nxt = smem + ((kt + 1) & 1) * STAGE_BYTES;
    constexpr bool DMA = !(ABL & ABL_NO_DMA), RD = !(ABL & ABL_NO_LDS_READ);
    if constexpr (LATE && DMA) {
      const int k1 = k_begin + (kt + 1) * BK;
      lp.template issue<2, 4, 510 + ABL>(nxt, wave, k1);
      lq.template issue<2, 4, 510 + ABL>(nxt + OPER_STAGE_BYTES, wave, k1);
    }
    if constexpr (RD) load_frags16x8(fb, cur + p_wave_off, cur + q_wave_off, off[1]);
    mma_frags16x8(acc, fa);
#pragma unroll
    for (int i = 0; i < 12; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
      if (LATE && i < 4) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, 8, 0);
    if constexpr (!(ABL & ABL_NO_BARRIER)) {
      asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
      __syncthreads();
    }
    if constexpr (AHEAD && DMA) {
      const int k2 = k_begin + (kt + 2) * BK;
      lp.template issue<0, 2, 520 + ABL>(cur, wave, k2);
      lq.template issue<0, 2, 520 + ABL>(cur + OPER_STAGE_BYTES, wave, k2);
    }
    // (after the last K-step this reads the idle stage: values nobody uses)
    if constexpr (RD) load_frags16x8(fa, nxt + p_wave_off, nxt + q_wave_off, off[0]);
    mma_frags16x8(acc, fb);
#pragma unroll
    for (int i = 0; i < 12; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
      if (AHEAD && i < 4) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, 8, 0);
  };
  using yes = std::integral_constant<bool, true>;
  using no = std::integral_constant<bool, false>;
  for (int kt = 0; kt < nk - 2; ++kt) k_step(kt, yes{}, yes{});
  if (nk > 1) k_step(nk - 2, yes{}, no{});
  k_step(nk - 1, no{}, no{});
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
  __syncthreads();
}

}  // namespace artk
