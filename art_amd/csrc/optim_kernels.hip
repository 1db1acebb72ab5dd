// Optimizer step for the LoRA parameters, gfx950.
//
// The reference trains the adapters with HF Trainer's `paged_adamw_8bit`
// (bitsandbytes) and `max_grad_norm = 0.1`, `weight_decay = 0.1`, betas
// (0.9, 0.99), constant learning rate (src/art/dev/model.py:69-85).  Here all
// adapter parameters of the model live in ONE flat fp32 buffer (likewise their
// gradients and the two moments), so a step is two launches over contiguous
// memory instead of several small kernels per tensor: a fixed-order sum of
// squares for the global gradient norm, and a fused update that applies the
// clip coefficient, the decoupled weight decay and the Adam update, and also
// writes the bf16 copy of the parameters that the GEMM kernels read.  Moments
// are fp32 (the reference quantises them to 8 bits block-wise; that is a memory
// optimisation of bitsandbytes, not part of the update rule).
// Both kernels are HBM-bound: 4 B/param and 16 B read + 14 B written per param.
#include "common.hpp"

namespace artk {

constexpr int SUMSQ_BLOCKS = 1024;

// part[b] = sum of x[i]^2 over the slice of block b, accumulated in double in a
// fixed order; sumsq_final_kernel adds the partials in index order.
__global__ __launch_bounds__(256) void sumsq_partial_kernel(const float* __restrict__ x, int64_t n,
                                                            double* __restrict__ part) {
  __shared__ double red[4];
  const int64_t per = ((n + SUMSQ_BLOCKS - 1) / SUMSQ_BLOCKS + 3) & ~(int64_t)3;
  const int64_t b0 = (int64_t)blockIdx.x * per;
  const int64_t b1 = b0 + per < n ? b0 + per : n;
  double acc = 0.0;
  for (int64_t i = b0 + threadIdx.x * 4; i < b1; i += 1024) {
    if (i + 4 <= b1 && ((uintptr_t)(x + i) & 15) == 0) {
      const float4 v = *(const float4*)(x + i);
      acc += (double)v.x * v.x + (double)v.y * v.y + (double)v.z * v.z + (double)v.w * v.w;
    } else {
      for (int64_t j = i; j < i + 4 && j < b1; ++j) acc += (double)x[j] * x[j];
    }
  }
  acc = wave_sum(acc);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = acc;
  __syncthreads();
  if (threadIdx.x == 0) part[blockIdx.x] = red[0] + red[1] + red[2] + red[3];
}

__global__ __launch_bounds__(64) void sumsq_final_kernel(const double* __restrict__ part,
                                                         float* __restrict__ out) {
  // lane l adds its 16 consecutive partials in index order, then a fixed butterfly over the wave
  double s = 0.0;
  for (int i = 0; i < SUMSQ_BLOCKS / 64; ++i) s += part[threadIdx.x * (SUMSQ_BLOCKS / 64) + i];
  s = wave_sum(s);
  if (threadIdx.x == 0) out[0] = (float)s;
}

struct AdamWParams {
  float* p;
  const float* g;
  float* m;
  float* v;
  uint16_t* p_bf16;         // or nullptr
  const float* grad_sumsq;  // or nullptr: no clipping
  int64_t n;
  float lr, beta1, beta2, eps, weight_decay, max_grad_norm;
  float step_size;          // lr / (1 - beta1^t)
  float inv_bc2_sqrt;       // 1 / sqrt(1 - beta2^t)
};

__device__ __forceinline__ float adamw_one(float& p, float g, float& m, float& v, const AdamWParams& a,
                                           float clip) {
  g *= clip;
  p *= 1.f - a.lr * a.weight_decay;
  m = m + (g - m) * (1.f - a.beta1);
  v = v * a.beta2 + (1.f - a.beta2) * g * g;
  const float denom = sqrtf(v) * a.inv_bc2_sqrt + a.eps;
  p -= a.step_size * (m / denom);
  return p;
}

__global__ __launch_bounds__(256) void adamw_kernel(AdamWParams a) {
  float clip = 1.f;
  if (a.grad_sumsq != nullptr) {
    // torch.nn.utils.clip_grad_norm_: coef = max_norm / (norm + 1e-6), clamped to 1
    const float c = a.max_grad_norm / (sqrtf(a.grad_sumsq[0]) + 1e-6f);
    clip = c < 1.f ? c : 1.f;
  }
  const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
  if (i >= a.n) return;
  if (i + 4 <= a.n) {
    float4 p = *(float4*)(a.p + i), m = *(float4*)(a.m + i), v = *(float4*)(a.v + i);
    const float4 g = *(const float4*)(a.g + i);
    adamw_one(p.x, g.x, m.x, v.x, a, clip);
    adamw_one(p.y, g.y, m.y, v.y, a, clip);
    adamw_one(p.z, g.z, m.z, v.z, a, clip);
    adamw_one(p.w, g.w, m.w, v.w, a, clip);
    *(float4*)(a.p + i) = p;
    *(float4*)(a.m + i) = m;
    *(float4*)(a.v + i) = v;
    if (a.p_bf16) {
      const uint32_t lo = (uint32_t)f32_to_bf16(p.x) | ((uint32_t)f32_to_bf16(p.y) << 16);
      const uint32_t hi = (uint32_t)f32_to_bf16(p.z) | ((uint32_t)f32_to_bf16(p.w) << 16);
      *(uint2*)(a.p_bf16 + i) = make_uint2(lo, hi);
    }
  } else {
    for (int64_t j = i; j < a.n; ++j) {
      float p = a.p[j], m = a.m[j], v = a.v[j];
      adamw_one(p, a.g[j], m, v, a, clip);
      a.p[j] = p;
      a.m[j] = m;
      a.v[j] = v;
      if (a.p_bf16) a.p_bf16[j] = f32_to_bf16(p);
    }
  }
}

// ----------------------------------------------------------------------------
// AdamW with 8-bit block-wise moments (the storage form of `paged_adamw_8bit`).
// Each moment is one byte per element: an index into a 256-entry code book of
// values in [-1, 1] (exp_avg) or [0, 1] (exp_avg_sq), times one fp32 absolute
// maximum per block of 256 elements.  One work-group = one block: dequantise,
// update in fp32, new block maxima, requantise to the nearest code.
// ----------------------------------------------------------------------------
struct AdamW8Params {
  float* p;
  const float* g;
  uint8_t* c1;
  uint8_t* c2;
  float* absmax1;
  float* absmax2;
  const float* qmap1;
  const float* qmap2;
  uint16_t* p_bf16;
  const float* grad_sumsq;
  int64_t n;
  float lr, beta1, beta2, eps, weight_decay, max_grad_norm;
  float step_size;   // -lr * sqrt(1 - beta2^t) / (1 - beta1^t)
  float eps_scaled;  // sqrt(1 - beta2^t) * eps
};

// Index of the entry of the ascending code book nearest to x (ties to the lower index).
__device__ __forceinline__ int nearest_code(const float* map, float x) {
  int lo = 0, hi = 255;  // invariant: map[lo] <= x (or lo == 0), map[hi] >= x (or hi == 255)
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (map[mid] <= x) lo = mid; else hi = mid;
  }
  return (x - map[lo] <= map[hi] - x) ? lo : hi;
}

__global__ __launch_bounds__(256) void adamw8bit_kernel(AdamW8Params a) {
  __shared__ float map1[256], map2[256];
  __shared__ float red[2][4];
  map1[threadIdx.x] = a.qmap1[threadIdx.x];
  map2[threadIdx.x] = a.qmap2[threadIdx.x];
  float clip = 1.f;
  if (a.grad_sumsq != nullptr) {
    const float c = a.max_grad_norm / (sqrtf(a.grad_sumsq[0]) + 1e-6f);
    clip = c < 1.f ? c : 1.f;
  }
  __syncthreads();
  const int64_t b = blockIdx.x;
  const int64_t i = b * 256 + threadIdx.x;
  const bool in = i < a.n;
  float m = 0.f, v = 0.f, g = 0.f, pv = 0.f;
  if (in) {
    g = a.g[i] * clip;
    pv = a.p[i];
    m = map1[a.c1[i]] * a.absmax1[b];
    v = map2[a.c2[i]] * a.absmax2[b];
    m = m * a.beta1 + (1.f - a.beta1) * g;
    v = v * a.beta2 + (1.f - a.beta2) * g * g;
  }
  float mx1 = wave_max(fabsf(m)), mx2 = wave_max(fabsf(v));
  if ((threadIdx.x & 63) == 0) {
    red[0][threadIdx.x >> 6] = mx1;
    red[1][threadIdx.x >> 6] = mx2;
  }
  __syncthreads();
  mx1 = fmaxf(fmaxf(red[0][0], red[0][1]), fmaxf(red[0][2], red[0][3]));
  mx2 = fmaxf(fmaxf(red[1][0], red[1][1]), fmaxf(red[1][2], red[1][3]));
  if (threadIdx.x == 0) {
    a.absmax1[b] = mx1;
    a.absmax2[b] = mx2;
  }
  if (!in) return;
  pv = pv + a.step_size * (m / (sqrtf(v) + a.eps_scaled));
  if (a.weight_decay > 0.f) pv = pv * (1.f - a.lr * a.weight_decay);
  a.p[i] = pv;
  if (a.p_bf16) a.p_bf16[i] = f32_to_bf16(pv);
  a.c1[i] = (uint8_t)nearest_code(map1, mx1 > 0.f ? m / mx1 : 0.f);
  a.c2[i] = (uint8_t)nearest_code(map2, mx2 > 0.f ? v / mx2 : 0.f);
}

}  // namespace artk

using namespace artk;

extern "C" {

size_t artk_sumsq_f32_workspace_bytes(void) { return SUMSQ_BLOCKS * sizeof(double) + 256; }

int32_t artk_sumsq_f32(const float* x, int64_t n, float* out, void* workspace, size_t workspace_bytes,
                       artk_stream_t stream) {
  ARTK_CHECK_ARG(x && out && n > 0, "null pointer or empty input");
  Workspace ws(workspace, workspace_bytes);
  double* part = ws.take<double>(SUMSQ_BLOCKS);
  if (!ws.ok()) {
    set_error("workspace too small: need %zu bytes, got %zu", ws.used, workspace_bytes);
    return ARTK_ERR_WORKSPACE_TOO_SMALL;
  }
  hipStream_t st = (hipStream_t)stream;
  sumsq_partial_kernel<<<SUMSQ_BLOCKS, 256, 0, st>>>(x, n, part);
  ARTK_CHECK_LAUNCH();
  sumsq_final_kernel<<<1, 64, 0, st>>>(part, out);
  ARTK_CHECK_LAUNCH();
  return ARTK_OK;
}

int32_t artk_adamw_step(float* params, const float* grads, float* exp_avg, float* exp_avg_sq,
                        void* params_bf16, int64_t n, float lr, float beta1, float beta2, float eps,
                        float weight_decay, int32_t step, const float* grad_sumsq, float max_grad_norm,
                        artk_stream_t stream) {
  ARTK_CHECK_ARG(params && grads && exp_avg && exp_avg_sq, "null pointer argument");
  ARTK_CHECK_ARG(n > 0 && step >= 1, "n must be positive and step >= 1");
  ARTK_CHECK_ARG(aligned16(params) && aligned16(grads) && aligned16(exp_avg) && aligned16(exp_avg_sq) &&
                     (params_bf16 == nullptr || (((uintptr_t)params_bf16) & 7) == 0),
                 "buffers must be 16-byte aligned (bf16 copy: 8-byte)");
  ARTK_CHECK_ARG(beta1 >= 0.f && beta1 < 1.f && beta2 >= 0.f && beta2 < 1.f, "betas must be in [0, 1)");
  AdamWParams a;
  a.p = params;
  a.g = grads;
  a.m = exp_avg;
  a.v = exp_avg_sq;
  a.p_bf16 = (uint16_t*)params_bf16;
  a.grad_sumsq = grad_sumsq;
  a.n = n;
  a.lr = lr;
  a.beta1 = beta1;
  a.beta2 = beta2;
  a.eps = eps;
  a.weight_decay = weight_decay;
  a.max_grad_norm = max_grad_norm;
  // bias corrections in double on the host, as torch computes them with Python floats
  const double bc1 = 1.0 - pow((double)beta1, (double)step);
  const double bc2 = 1.0 - pow((double)beta2, (double)step);
  a.step_size = (float)((double)lr / bc1);
  a.inv_bc2_sqrt = (float)(1.0 / sqrt(bc2));
  const int64_t n4 = (n + 3) / 4;
  adamw_kernel<<<(unsigned)((n4 + 255) / 256), 256, 0, (hipStream_t)stream>>>(a);
  ARTK_CHECK_LAUNCH();
  return ARTK_OK;
}

int32_t artk_adamw8bit_step(float* params, const float* grads, void* state1, void* state2, float* absmax1,
                            float* absmax2, const float* qmap1, const float* qmap2, void* params_bf16,
                            int64_t n, float lr, float beta1, float beta2, float eps, float weight_decay,
                            int32_t step, const float* grad_sumsq, float max_grad_norm,
                            artk_stream_t stream) {
  ARTK_CHECK_ARG(params && grads && state1 && state2 && absmax1 && absmax2 && qmap1 && qmap2,
                 "null pointer argument");
  ARTK_CHECK_ARG(n > 0 && step >= 1, "n must be positive and step >= 1");
  ARTK_CHECK_ARG(beta1 >= 0.f && beta1 < 1.f && beta2 >= 0.f && beta2 < 1.f, "betas must be in [0, 1)");
  AdamW8Params a;
  a.p = params;
  a.g = grads;
  a.c1 = (uint8_t*)state1;
  a.c2 = (uint8_t*)state2;
  a.absmax1 = absmax1;
  a.absmax2 = absmax2;
  a.qmap1 = qmap1;
  a.qmap2 = qmap2;
  a.p_bf16 = (uint16_t*)params_bf16;
  a.grad_sumsq = grad_sumsq;
  a.n = n;
  a.lr = lr;
  a.beta1 = beta1;
  a.beta2 = beta2;
  a.eps = eps;
  a.weight_decay = weight_decay;
  a.max_grad_norm = max_grad_norm;
  const double c1 = 1.0 - pow((double)beta1, (double)step);
  const double c2 = sqrt(1.0 - pow((double)beta2, (double)step));
  a.step_size = (float)(-(double)lr * c2 / c1);
  a.eps_scaled = (float)(c2 * (double)eps);
  adamw8bit_kernel<<<(unsigned)((n + 255) / 256), 256, 0, (hipStream_t)stream>>>(a);
  ARTK_CHECK_LAUNCH();
  return ARTK_OK;
}

}  // extern "C"
