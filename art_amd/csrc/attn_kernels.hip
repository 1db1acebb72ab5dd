// Packed-row attention for gfx950 (MI355X, CDNA4).
//
// The reference materialises a dense [1,S,S] additive bias from the packed
// row's ids (src/art/local/train.py:177-215):
//     visible(i, j) = j <= i && (group[i] == group[j] || parent[i] == group[j])
// and passes it to the model as `causal_mask` (train.py:239-241).  Here the
// matrix is never built.  A plan (once per packed row, shared by every layer
// and head) turns the 64-bit ids into int32 equality codes and classifies each
// (query block, key block) pair as invisible / partly visible / fully visible;
// the attention kernels walk only the visible blocks and evaluate the rule per
// element only in the partly visible ones.
//
// Forward work-group: 256 queries x one head, 8 wavefronts of 32 queries, key
// tiles of 64.  Scores are computed transposed (S^T = K Q^T, MFMA 32x32x16), so
// that a lane owns one query: the row maximum and sum are in-lane reductions
// plus one exchange between the two half-waves, the accumulator of S^T is
// already in the B-operand layout of the second product O^T = V^T P^T, and the
// running rescale of O^T is a per-lane scalar.  K tiles ([key][d]) and V^T
// tiles ([d][key], from a transposed copy of V made once per call) are brought
// into a 3-stage LDS ring by buffer_load ... lds.
#include "common.hpp"
#include "gemm_nt.hpp"

namespace artk {

constexpr int ATT_BM = 256;    // queries per work-group
constexpr int ATT_BN = 64;     // keys per tile
constexpr int ATT_STAGES = 3;
constexpr int ATT_MAX_KB = 1024;  // key blocks per row the list in LDS can hold

// ----------------------------------------------------------------------------
// Plan
// ----------------------------------------------------------------------------

// gc[t] = first position whose group id equals group_ids[t];
// pc[t] = first position whose group id equals parent_ids[t], or -2 if none.
// Then group[i] == group[j] <=> gc[i] == gc[j] and parent[i] == group[j] <=>
// pc[i] == gc[j].  Brute force over all pairs (integer work, once per row).
__global__ __launch_bounds__(256) void attn_codes_kernel(const int64_t* __restrict__ group_ids,
                                                         const int64_t* __restrict__ parent_ids,
                                                         int S, int* __restrict__ gc,
                                                         int* __restrict__ pc) {
  __shared__ int64_t tile[256];
  const int t = blockIdx.x * 256 + threadIdx.x;
  const int64_t g = t < S ? group_ids[t] : 0;
  const int64_t pa = t < S ? parent_ids[t] : 0;
  int first_g = 0x7fffffff, first_p = 0x7fffffff;
  for (int j0 = 0; j0 < S; j0 += 256) {
    __syncthreads();
    tile[threadIdx.x] = j0 + (int)threadIdx.x < S ? group_ids[j0 + threadIdx.x] : 0;
    __syncthreads();
    const int lim = S - j0 < 256 ? S - j0 : 256;
    for (int jj = 0; jj < lim; ++jj) {
      const int64_t id = tile[jj];
      if (id == g && j0 + jj < first_g) first_g = j0 + jj;
      if (id == pa && j0 + jj < first_p) first_p = j0 + jj;
    }
  }
  if (t < S) {
    gc[t] = first_g;
    pc[t] = first_p == 0x7fffffff ? -2 : first_p;
  }
}

__device__ __forceinline__ bool attn_visible(int i, int j, int gi, int pi, int gj) {
  return j <= i && (gj == gi || gj == pi);
}

// cls[qb][kb] for query blocks of BM and key blocks of BN positions:
// 0 = no visible pair, 1 = some, 2 = all BM*BN pairs.  clsT is the transpose.
// One wavefront per (qb, kb).
__global__ __launch_bounds__(256) void attn_classify_kernel(const int* __restrict__ gc,
                                                            const int* __restrict__ pc, int BM,
                                                            int BN, int nQb, int nKb,
                                                            uint8_t* __restrict__ cls,
                                                            uint8_t* __restrict__ clsT) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int kb = blockIdx.x * 4 + wave;
  const int qb = blockIdx.y;
  if (kb >= nKb) return;
  int total = 0;
  if (kb * BN <= qb * BM + BM - 1) {
    int cnt = 0;
    for (int kk = lane; kk < BN; kk += 64) {
      const int j = kb * BN + kk;
      const int gj = gc[j];
      for (int ii = 0; ii < BM; ++ii) {
        const int i = qb * BM + ii;
        cnt += attn_visible(i, j, gc[i], pc[i], gj) ? 1 : 0;
      }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) cnt += __shfl_xor(cnt, o, 64);
    total = cnt;
  }
  if (lane == 0) {
    const uint8_t c = total == 0 ? 0 : (total == BM * BN ? 2 : 1);
    cls[(int64_t)qb * nKb + kb] = c;
    if (clsT) clsT[(int64_t)kb * nQb + qb] = c;
  }
}

// list[row][0..cnt[row]) = the columns of cls[row][*] that are not 0, ascending,
// as  column | class << 14.  One work-group per row.
__global__ __launch_bounds__(256) void attn_compact_kernel(const uint8_t* __restrict__ cls,
                                                           int ncol, uint16_t* __restrict__ list,
                                                           int* __restrict__ cnt) {
  __shared__ int wtot[4];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int row = blockIdx.x;
  int base = 0;
  for (int c0 = 0; c0 < ncol; c0 += 256) {
    const int c = c0 + threadIdx.x;
    const int v = c < ncol ? cls[(int64_t)row * ncol + c] : 0;
    const unsigned long long m = __ballot(v != 0);
    const int rank = __popcll(m & ((1ull << lane) - 1ull));
    __syncthreads();
    if (lane == 0) wtot[wave] = __popcll(m);
    __syncthreads();
    int off = base;
    for (int w = 0; w < wave; ++w) off += wtot[w];
    if (v) list[(int64_t)row * ncol + off + rank] = (uint16_t)(c | (v << 14));
    base += wtot[0] + wtot[1] + wtot[2] + wtot[3];
  }
  if (threadIdx.x == 0) cnt[row] = base;
}

// Device-memory layout of a plan for a row of S positions (S % 256 == 0).
struct AttnPlan {
  int* gc;
  int* pc;
  int nQb, nKb;        // forward: query blocks of 256, key blocks of 64
  uint8_t* cls;        // [nQb][nKb]
  uint16_t* list;      // [nQb][nKb]
  int* cnt;            // [nQb]
  int nQb2, nKb2;      // backward: query blocks of 64 / key blocks of 256 (see the backward kernels)
  uint8_t* cls2;       // [nQb2][nKb2]
  uint8_t* cls2T;      // [nKb2][nQb2]
  uint16_t* list_q;    // per query block (dQ kernel): reuses cls/list above
  uint16_t* list2T;    // [nKb2][nQb2] query blocks per key block
  int* cnt2T;          // [nKb2]
};

static size_t attn_plan_layout(void* base, size_t bytes, int64_t S, AttnPlan& pl) {
  Workspace ws(base, bytes);
  pl.nQb = (int)(S / ATT_BM);
  pl.nKb = (int)(S / ATT_BN);
  pl.nQb2 = (int)(S / ATT_BN);
  pl.nKb2 = (int)(S / ATT_BM);
  pl.gc = ws.take<int>((size_t)S);
  pl.pc = ws.take<int>((size_t)S);
  pl.cls = ws.take<uint8_t>((size_t)pl.nQb * pl.nKb);
  pl.list = ws.take<uint16_t>((size_t)pl.nQb * pl.nKb);
  pl.cnt = ws.take<int>((size_t)pl.nQb);
  pl.cls2 = ws.take<uint8_t>((size_t)pl.nQb2 * pl.nKb2);
  pl.cls2T = ws.take<uint8_t>((size_t)pl.nQb2 * pl.nKb2);
  pl.list2T = ws.take<uint16_t>((size_t)pl.nQb2 * pl.nKb2);
  pl.cnt2T = ws.take<int>((size_t)pl.nKb2);
  pl.list_q = pl.list;
  return ws.ok() || base == nullptr ? ws.used : (size_t)-1;
}

// ----------------------------------------------------------------------------
// Transposed copy of one operand: out[h][d][s] = in[s * ss + h * hs + d]
// ----------------------------------------------------------------------------
__global__ __launch_bounds__(256) void attn_transpose_kernel(const uint16_t* __restrict__ in,
                                                             int64_t ss, int64_t hs, int S, int D,
                                                             uint16_t* __restrict__ out) {
  __shared__ uint16_t tile[64][66];
  const int s0 = blockIdx.x * 64, d0 = blockIdx.y * 64, hd = blockIdx.z;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int i = ty; i < 64; i += 4) {
    const int s = s0 + i, d = d0 + tx;
    tile[i][tx] = (s < S && d < D) ? in[(int64_t)s * ss + (int64_t)hd * hs + d] : (uint16_t)0;
  }
  __syncthreads();
  for (int i = ty; i < 64; i += 4) {
    const int d = d0 + i, s = s0 + tx;
    if (d < D && s < S) out[((int64_t)hd * D + d) * S + s] = tile[tx][i];
  }
}

// ----------------------------------------------------------------------------
// Forward
// ----------------------------------------------------------------------------
struct AttnFwdParams {
  const uint16_t* Q;   // element (s, h, d) at s * q_ss + h * q_hs + d
  const uint16_t* K;
  const uint16_t* Vt;  // [Hkv][D][S]
  uint16_t* O;
  float* lse;          // [Hq][S], natural log
  int64_t q_ss, q_hs, k_ss, k_hs, o_ss, o_hs;
  const int* gc;
  const int* pc;
  const uint16_t* list;
  const int* cnt;
  int S, Hq, Hkv, nQb, nKb;
  float scale_log2e;
};

template <int D>
struct AttnTile {
  static constexpr int CHK = D / 8;                    // 16-byte chunks of a K row
  static constexpr int K_BYTES = ATT_BN * D * 2;
  static constexpr int V_BYTES = D * ATT_BN * 2;
  static constexpr int CODE_OFF = K_BYTES + V_BYTES;
  static constexpr int STAGE = CODE_OFF + 1024;
  static constexpr int NK = K_BYTES / 1024 / 8;        // DMA instructions per wave (8 waves)
  static constexpr int NV = V_BYTES / 1024 / 8;
  static constexpr int N_PER = NK + NV + 1;
  // chunk swizzle: K rows of D*2 bytes, V^T rows of 128 bytes
  __device__ static __forceinline__ int swz_k(int row) {
    return CHK == 16 ? (row & 15) : ((row >> 1) & 7);
  }
  __device__ static __forceinline__ int swz_v(int row) { return (row >> 1) & 7; }
};

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// DMA of key block kb into one LDS stage: this wave's share of the K tile and of
// the V^T tile, plus the 64 key codes (every wave writes the same 256 bytes).
template <int D>
__device__ __forceinline__ void attn_issue(char* st, int kb, __amdgpu_buffer_rsrc_t rsrc_k,
                                           __amdgpu_buffer_rsrc_t rsrc_v,
                                           __amdgpu_buffer_rsrc_t rsrc_c,
                                           const int (&voff_k)[AttnTile<D>::NK],
                                           const int (&voff_v)[AttnTile<D>::NV], int64_t k_ss,
                                           int wave, int lane) {
  using T = AttnTile<D>;
  const int k0 = kb * ATT_BN;
#pragma unroll
  for (int i = 0; i < T::NK; ++i)
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_k, (lds_ptr_t)(st + (wave * T::NK + i) * 1024), 16,
                                             voff_k[i], (int)(k0 * k_ss * 2), 0, 0);
#pragma unroll
  for (int i = 0; i < T::NV; ++i)
    __builtin_amdgcn_raw_ptr_buffer_load_lds(
        rsrc_v, (lds_ptr_t)(st + T::K_BYTES + (wave * T::NV + i) * 1024), 16, voff_v[i], k0 * 2, 0, 0);
  __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_c, (lds_ptr_t)(st + T::CODE_OFF), 4, lane * 4, k0 * 4, 0,
                                           0);
}

template <int D>
__global__ __launch_bounds__(512) void attn_fwd_kernel(AttnFwdParams p) {
  using T = AttnTile<D>;
  __shared__ __attribute__((aligned(1024))) char smem[ATT_STAGES * T::STAGE];
  __shared__ uint16_t s_list[ATT_MAX_KB];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n = lane & 31, h = lane >> 5;
  const int hq = blockIdx.x % p.Hq;
  const int qb = p.nQb - 1 - (int)(blockIdx.x / p.Hq);  // long rows first
  const int hkv = hq / (p.Hq / p.Hkv);
  const int q = qb * ATT_BM + wave * 32 + n;
  const int cnt = p.cnt[qb];

  for (int i = threadIdx.x; i < cnt; i += 512) s_list[i] = p.list[(int64_t)qb * p.nKb + i];

  // this lane's query as B-operand fragments of S^T = K Q^T
  bf16x8 qf[D / 16];
  {
    const uint16_t* qp = p.Q + (int64_t)q * p.q_ss + (int64_t)hq * p.q_hs + 8 * h;
#pragma unroll
    for (int s = 0; s < D / 16; ++s) qf[s] = *(const bf16x8*)(qp + 16 * s);
  }
  const int gi = p.gc[q], pi = p.pc[q];

  const __amdgpu_buffer_rsrc_t rsrc_k = __builtin_amdgcn_make_buffer_rsrc(
      (void*)(p.K + (int64_t)hkv * p.k_hs), 0, 0x7fffffff, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_v = __builtin_amdgcn_make_buffer_rsrc(
      (void*)(p.Vt + (int64_t)hkv * D * p.S), 0, 0x7fffffff, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_c =
      __builtin_amdgcn_make_buffer_rsrc((void*)p.gc, 0, 0x7fffffff, 0x00020000);
  int voff_k[T::NK], voff_v[T::NV];
#pragma unroll
  for (int i = 0; i < T::NK; ++i) {
    const int r = (wave * T::NK + i) * (64 / T::CHK) + lane / T::CHK;
    const int c = (lane % T::CHK) ^ T::swz_k(r);
    voff_k[i] = (int)(r * p.k_ss * 2) + c * 16;
  }
#pragma unroll
  for (int i = 0; i < T::NV; ++i) {
    const int r = (wave * T::NV + i) * 8 + lane / 8;
    const int c = (lane % 8) ^ T::swz_v(r);
    voff_v[i] = r * p.S * 2 + c * 16;
  }
  __syncthreads();  // s_list

  auto* list_lds = s_list;
#define ATTN_ISSUE(IT, STG) \
  attn_issue<D>(smem + (STG) * T::STAGE, __builtin_amdgcn_readfirstlane(list_lds[IT] & 0x3fff), rsrc_k, \
                rsrc_v, rsrc_c, voff_k, voff_v, p.k_ss, wave, lane)

  floatx16 o[D / 32];
#pragma unroll
  for (int dt = 0; dt < D / 32; ++dt)
#pragma unroll
    for (int j = 0; j < 16; ++j) o[dt][j] = 0.f;
  float m_run = -1e30f, l_run = 0.f;

  if (cnt > 0) ATTN_ISSUE(0, 0);
  if (cnt > 1) ATTN_ISSUE(1, 1);
  int stage = 0;
  for (int it = 0; it < cnt; ++it) {
    if (it + 1 < cnt)
      wait_vmcnt<T::N_PER>();
    else
      wait_vmcnt<0>();
    __syncthreads();
    if (it + 2 < cnt) ATTN_ISSUE(it + 2, stage >= 1 ? stage - 1 : ATT_STAGES - 1);
    const int entry = __builtin_amdgcn_readfirstlane(s_list[it]);
    const int kb = entry & 0x3fff;
    const bool partial = (entry >> 14) == 1;
    const char* st = smem + stage * T::STAGE;

    // S^T tiles: keys 0..31 and 32..63 of the block x this wave's 32 queries
    floatx16 sc[2];
#pragma unroll
    for (int j = 0; j < 16; ++j) sc[0][j] = sc[1][j] = 0.f;
#pragma unroll
    for (int s = 0; s < D / 16; ++s) {
#pragma unroll
      for (int kt = 0; kt < 2; ++kt) {
        const int row = 32 * kt + n;
        const bf16x8 a = *(const bf16x8*)(st + row * (D * 2) + (((2 * s + h) ^ T::swz_k(row)) * 16));
        sc[kt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qf[s], sc[kt], 0, 0, 0);
      }
    }

    // scale, mask, running max
    float mloc = -INFINITY;
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int j = 0; j < 16; ++j) sc[kt][j] *= p.scale_log2e;
    if (partial) {
      const int* codes = (const int*)(st + T::CODE_OFF);
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) {
          const int kk = 32 * kt + 8 * g4 + 4 * h;
          const int4 kc = *(const int4*)(codes + kk);
          const int key = kb * ATT_BN + kk;
          const int kcv[4] = {kc.x, kc.y, kc.z, kc.w};
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (!attn_visible(q, key + e, gi, pi, kcv[e])) sc[kt][4 * g4 + e] = -INFINITY;
        }
    }
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int j = 0; j < 16; ++j) mloc = fmaxf(mloc, sc[kt][j]);
    mloc = fmaxf(mloc, __shfl_xor(mloc, 32, 64));
    const float m_new = fmaxf(m_run, mloc);
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
    m_run = m_new;
    float lsum = 0.f;
    bf16x8 pf[4];
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        const float e = __builtin_amdgcn_exp2f(sc[kt][j] - m_new);
        lsum += e;
        pf[2 * kt + j / 8][j % 8] = (__bf16)e;
      }
    l_run = l_run * alpha + lsum;
    if (__any(alpha != 1.f)) {
#pragma unroll
      for (int dt = 0; dt < D / 32; ++dt)
#pragma unroll
        for (int j = 0; j < 16; ++j) o[dt][j] *= alpha;
    }

    // O^T += V^T P^T
    const char* vt = st + T::K_BYTES;
#pragma unroll
    for (int s2 = 0; s2 < 4; ++s2) {
#pragma unroll
      for (int dt = 0; dt < D / 32; ++dt) {
        const int row = 32 * dt + n;
        const int sw = T::swz_v(row);
        const bf16x4 lo = *(const bf16x4*)(vt + row * 128 + (((2 * s2) ^ sw) * 16) + 8 * h);
        const bf16x4 hi = *(const bf16x4*)(vt + row * 128 + (((2 * s2 + 1) ^ sw) * 16) + 8 * h);
        const bf16x8 a = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, pf[s2], o[dt], 0, 0, 0);
      }
    }
    stage = stage + 1 == ATT_STAGES ? 0 : stage + 1;
  }

  const float l_tot = l_run + __shfl_xor(l_run, 32, 64);
  const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
  uint16_t* op = p.O + (int64_t)q * p.o_ss + (int64_t)hq * p.o_hs + 4 * h;
#pragma unroll
  for (int dt = 0; dt < D / 32; ++dt)
#pragma unroll
    for (int g4 = 0; g4 < 4; ++g4) {
      bf16x4 v;
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = (__bf16)(o[dt][4 * g4 + e] * inv);
      *(bf16x4*)(op + 32 * dt + 8 * g4) = v;
    }
  if (h == 0) p.lse[(int64_t)hq * p.S + q] = (m_run + __builtin_amdgcn_logf(l_tot)) * LN2;
#undef ATTN_ISSUE
}

}  // namespace artk

using namespace artk;

extern "C" {

size_t artk_attn_plan_bytes(int64_t S) {
  AttnPlan pl;
  return attn_plan_layout(nullptr, 0, S, pl) + 256;
}

int32_t artk_attn_plan(const int64_t* group_ids, const int64_t* parent_ids, int64_t S, void* plan,
                       size_t plan_bytes, artk_stream_t stream) {
  ARTK_CHECK_ARG(group_ids && parent_ids && plan, "null pointer argument");
  ARTK_CHECK_ARG(S > 0, "S must be positive");
  if (S % ATT_BM != 0 || S / ATT_BN > ATT_MAX_KB) {
    set_error("row length %lld must be a multiple of %d and at most %d", (long long)S, ATT_BM,
              ATT_MAX_KB * ATT_BN);
    return ARTK_ERR_UNSUPPORTED_SHAPE;
  }
  AttnPlan pl;
  if (attn_plan_layout(plan, plan_bytes, S, pl) == (size_t)-1) {
    set_error("plan buffer too small: need %zu bytes, got %zu", artk_attn_plan_bytes(S), plan_bytes);
    return ARTK_ERR_WORKSPACE_TOO_SMALL;
  }
  hipStream_t st = (hipStream_t)stream;
  attn_codes_kernel<<<(unsigned)(S / 256), 256, 0, st>>>(group_ids, parent_ids, (int)S, pl.gc, pl.pc);
  ARTK_CHECK_LAUNCH();
  attn_classify_kernel<<<dim3((unsigned)((pl.nKb + 3) / 4), (unsigned)pl.nQb), 256, 0, st>>>(
      pl.gc, pl.pc, ATT_BM, ATT_BN, pl.nQb, pl.nKb, pl.cls, nullptr);
  ARTK_CHECK_LAUNCH();
  attn_compact_kernel<<<(unsigned)pl.nQb, 256, 0, st>>>(pl.cls, pl.nKb, pl.list, pl.cnt);
  ARTK_CHECK_LAUNCH();
  attn_classify_kernel<<<dim3((unsigned)((pl.nKb2 + 3) / 4), (unsigned)pl.nQb2), 256, 0, st>>>(
      pl.gc, pl.pc, ATT_BN, ATT_BM, pl.nQb2, pl.nKb2, pl.cls2, pl.cls2T);
  ARTK_CHECK_LAUNCH();
  attn_compact_kernel<<<(unsigned)pl.nKb2, 256, 0, st>>>(pl.cls2T, pl.nQb2, pl.list2T, pl.cnt2T);
  ARTK_CHECK_LAUNCH();
  return ARTK_OK;
}

static int32_t attn_check(int64_t S, int32_t Hq, int32_t Hkv, int32_t D, const int64_t* strides,
                          int nstrides) {
  ARTK_CHECK_ARG(S > 0 && Hq > 0 && Hkv > 0, "S, Hq, Hkv must be positive");
  if (S % ATT_BM != 0 || S / ATT_BN > ATT_MAX_KB) {
    set_error("row length %lld must be a multiple of %d and at most %d", (long long)S, ATT_BM,
              ATT_MAX_KB * ATT_BN);
    return ARTK_ERR_UNSUPPORTED_SHAPE;
  }
  if (D != 64 && D != 128) {
    set_error("head dimension %d is not supported (64 or 128)", D);
    return ARTK_ERR_UNSUPPORTED_SHAPE;
  }
  if (Hq % Hkv != 0) {
    set_error("query heads (%d) must be a multiple of key/value heads (%d)", Hq, Hkv);
    return ARTK_ERR_UNSUPPORTED_SHAPE;
  }
  for (int i = 0; i < nstrides; ++i) {
    ARTK_CHECK_ARG(strides[i] > 0 && strides[i] % 8 == 0, "strides must be positive multiples of 8 elements");
    ARTK_CHECK_ARG(i % 2 != 0 || S * strides[i] * 2 < (1ll << 31), "operand spans 2 GiB or more");
  }
  return ARTK_OK;
}

size_t artk_attn_fwd_workspace_bytes(int64_t S, int32_t Hkv, int32_t D) {
  Workspace ws(nullptr, 0);
  ws.take<uint16_t>((size_t)S * Hkv * D);
  return ws.used + 256;
}

int32_t artk_attn_fwd(const void* q, const void* k, const void* v, const void* plan, int64_t S,
                      int32_t Hq, int32_t Hkv, int32_t D, int64_t q_stride_s, int64_t q_stride_h,
                      int64_t k_stride_s, int64_t k_stride_h, int64_t v_stride_s, int64_t v_stride_h,
                      int64_t o_stride_s, int64_t o_stride_h, float scale, void* out, float* lse,
                      void* workspace, size_t workspace_bytes, artk_stream_t stream) {
  ARTK_CHECK_ARG(q && k && v && plan && out && lse, "null pointer argument");
  ARTK_CHECK_ARG(aligned16(q) && aligned16(k) && aligned16(v) && aligned16(out),
                 "q, k, v, out must be 16-byte aligned");
  const int64_t strides[8] = {q_stride_s, q_stride_h, k_stride_s, k_stride_h,
                              v_stride_s, v_stride_h, o_stride_s, o_stride_h};
  int32_t rc = attn_check(S, Hq, Hkv, D, strides, 8);
  if (rc) return rc;
  Workspace ws(workspace, workspace_bytes);
  uint16_t* vt = ws.take<uint16_t>((size_t)S * Hkv * D);
  if (!ws.ok()) {
    set_error("workspace too small: need %zu bytes, got %zu", ws.used, workspace_bytes);
    return ARTK_ERR_WORKSPACE_TOO_SMALL;
  }
  AttnPlan pl;
  attn_plan_layout(const_cast<void*>(plan), (size_t)1 << 40, S, pl);
  hipStream_t st = (hipStream_t)stream;
  attn_transpose_kernel<<<dim3((unsigned)(S / 64), (unsigned)(D / 64), (unsigned)Hkv), 256, 0, st>>>(
      (const uint16_t*)v, v_stride_s, v_stride_h, (int)S, D, vt);
  ARTK_CHECK_LAUNCH();
  AttnFwdParams p;
  p.Q = (const uint16_t*)q;
  p.K = (const uint16_t*)k;
  p.Vt = vt;
  p.O = (uint16_t*)out;
  p.lse = lse;
  p.q_ss = q_stride_s;
  p.q_hs = q_stride_h;
  p.k_ss = k_stride_s;
  p.k_hs = k_stride_h;
  p.o_ss = o_stride_s;
  p.o_hs = o_stride_h;
  p.gc = pl.gc;
  p.pc = pl.pc;
  p.list = pl.list;
  p.cnt = pl.cnt;
  p.S = (int)S;
  p.Hq = Hq;
  p.Hkv = Hkv;
  p.nQb = pl.nQb;
  p.nKb = pl.nKb;
  p.scale_log2e = scale * LOG2E;
  const unsigned grid = (unsigned)(pl.nQb * Hq);
  prof_begin(PROF_ATTN_FWD, st);
  if (D == 128)
    attn_fwd_kernel<128><<<grid, 512, 0, st>>>(p);
  else
    attn_fwd_kernel<64><<<grid, 512, 0, st>>>(p);
  prof_end(PROF_ATTN_FWD, st);
  ARTK_CHECK_LAUNCH();
  return ARTK_OK;
}

}  // extern "C"
