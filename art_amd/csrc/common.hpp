// Shared host/device helpers for the artk C-ABI library (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "../../include/artk.h"

namespace artk {

// ---- error reporting (thread-local message, integer return codes) ----------
void set_error(const char* fmt, ...);

#define ARTK_CHECK_ARG(cond, ...)         \
  do {                                    \
    if (!(cond)) {                        \
      artk::set_error(__VA_ARGS__);       \
      return ARTK_ERR_INVALID_ARGUMENT;   \
    }                                     \
  } while (0)

#define ARTK_CHECK_HIP(expr)                                                        \
  do {                                                                              \
    hipError_t e__ = (expr);                                                        \
    if (e__ != hipSuccess) {                                                        \
      artk::set_error("%s failed: %s", #expr, hipGetErrorString(e__));              \
      return (int32_t)e__;                                                          \
    }                                                                               \
  } while (0)

#define ARTK_CHECK_LAUNCH()                                                         \
  do {                                                                              \
    hipError_t e__ = hipGetLastError();                                             \
    if (e__ != hipSuccess) {                                                        \
      artk::set_error("kernel launch failed at %s:%d: %s", __FILE__, __LINE__,      \
                      hipGetErrorString(e__));                                      \
      return (int32_t)e__;                                                          \
    }                                                                               \
  } while (0)

static inline bool aligned16(const void* p) { return (((uintptr_t)p) & 15) == 0; }
static inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

// Bump allocator over a caller-provided workspace.
struct Workspace {
  char* base;
  size_t size;
  size_t used;
  Workspace(void* p, size_t n) : base((char*)p), size(n), used(0) {}
  // Returns nullptr when the workspace is exhausted (or absent while sizing).
  template <typename T>
  T* take(size_t count) {
    size_t off = align_up(used, 256);
    used = off + count * sizeof(T);
    if (base == nullptr || used > size) return nullptr;
    return (T*)(base + off);
  }
  bool ok() const { return base != nullptr && used <= size; }
};

// ---- optional per-kernel timing with HIP events on the launch stream ---------
// Off by default. When on, the launch helpers bracket each dominant kernel with
// two events; artk_profile_collect() (after the caller synchronised) sums them.
enum ProfKind { PROF_LMHEAD_FWD = 0, PROF_DHIDDEN_GEMM = 1, PROF_TARGET_REF = 2,
                PROF_LORA_GEMM = 3, PROF_MOE_GEMM = 4, PROF_ATTN_FWD = 5, PROF_ATTN_BWD_KV = 6,
                PROF_ATTN_BWD_Q = 7, PROF_KINDS = 8 };
void prof_begin(int kind, hipStream_t st);
void prof_end(int kind, hipStream_t st);

// ---- device helpers ---------------------------------------------------------
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
__device__ __forceinline__ double wave_sum(double v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}

__device__ __forceinline__ float bf16_to_f32(uint16_t b) { return __uint_as_float(((uint32_t)b) << 16); }
__device__ __forceinline__ uint16_t f32_to_bf16(float f) {
  __bf16 h = (__bf16)f;  // round-to-nearest-even (v_cvt_pk_bf16_f32 on gfx950)
  return __builtin_bit_cast(uint16_t, h);
}

constexpr float LOG2E = 1.4426950408889634f;
constexpr float LN2 = 0.6931471805599453f;

// Work-group barrier that waits for this wave's LDS traffic only.  __syncthreads() also carries a
// fence, for which the compiler drains every outstanding memory operation first (s_waitcnt
// vmcnt(0)): that would serialise the DMA ring, whose completion is tracked by hand here.
__device__ __forceinline__ void barrier_lds_only() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}


// LDS DMA (buffer_load ... lds: 64 lanes x 16 or 4 bytes land at lds_addr + 16 / 4 lane) issued
// from inline assembly.  Issued through the builtin, the compiler knows that LDS is written
// behind its back and puts s_waitcnt vmcnt(..) in front of later LDS reads, down to vmcnt(0)
// once per loop iteration, which drains a multi-stage ring; kernels that track the completion
// by hand (s_waitcnt vmcnt(n) before the barrier that publishes a stage) keep the instruction
// out of its sight.  Invisible operations only make the compiler's own waits stricter; the
// hand-written counts must not have other vector memory operations between issue and wait.
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t dma_rsrc_t;
__device__ __forceinline__ dma_rsrc_t dma_make_rsrc(const void* base, uint32_t bytes) {
  const uint64_t a = (uint64_t)base;
  return dma_rsrc_t{(uint32_t)a, (uint32_t)(a >> 32) & 0xffffu, bytes, 0x00020000u};
}
__device__ __forceinline__ void dma_load16(dma_rsrc_t rsrc, int voff, int soff, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
               :
               : "s"(lds_addr), "v"(voff), "s"(rsrc), "s"(soff)
               : "memory", "m0");
}
__device__ __forceinline__ void dma_load4(dma_rsrc_t rsrc, int voff, int soff, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dword %1, %2, %3 offen lds"
               :
               : "s"(lds_addr), "v"(voff), "s"(rsrc), "s"(soff)
               : "memory", "m0");
}
__device__ __forceinline__ uint32_t lds_addr_of(const void* p) {
  return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void*)p;
}

}  // namespace artk
