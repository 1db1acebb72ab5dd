// One-pass skinny products of the LoRA backward (shared by the plain and the grouped, per-expert
// LoRA linears): see lora_stats_kernel.
#pragma once
#include "common.hpp"
#include "gemm_nt.hpp"
#include "lora_common.hpp"

#include <type_traits>

namespace artk {

// ----------------------------------------------------------------------------
// Both skinny products of the backward in ONE pass over a [T,C] bf16 matrix X:
//   ROW  rp[chunk][t][e] = sum_{c in chunk} X[t,c] F[e,c]      F bf16 [R,C]  (g B: F = B^T)
//   COL  cp[slab][c][e]  = sum_{t in slab}  X[t,c] Y[t,e]      Y f32 [T,R]   (dB: Y = x A^T)
// A work-group owns a slab of rows x a chunk of columns and streams it through LDS
// in 128 x 128 tiles (buffer_load ... lds, three stages in flight), so X is read
// from HBM once, fully coalesced, for both products.  Both run on MFMA 32x32x16
// with the small dimension e as the M operand: ROW contracts over the columns
// (row fragments of the tile, ds_read_b128), COL over the rows (transposed
// fragments, ds_read_b64_tr_b16; Y of the row tile is staged as bf16, transposed).
// Wave w owns rows 32w.. of a tile for ROW and columns 32w.. for COL: no exchange
// between waves.  Partials over chunks / slabs are summed in a fixed order by
// stats_reduce_kernel.
// ----------------------------------------------------------------------------
constexpr int ST_TILE = 128;
constexpr int ST_ROW_BYTES = ST_TILE * 2;             // 256
constexpr int ST_TILE_BYTES = ST_TILE * ST_ROW_BYTES;  // 32 KiB
constexpr int ST_STAGES = 3;

struct StatsParams {
  const uint16_t* X;
  int64_t T, C;
  const uint16_t* F;  // [R,C] or nullptr: no ROW product
  const float* Y;     // [T,R] or nullptr: no COL product
  float* row_part;    // [n_chunks][T][R]
  float* col_part;    // [n_slabs][C][R]
  float* row_dummy;   // 1024 floats that out-of-range lanes of a ROW flush write to
  int R, rows_per_slab, n_slabs, n_chunks;
  int cc;  // columns per chunk: a multiple of 128, at most the kernel's NCT * 128
  // Grouped form (offsets != nullptr): slab s is the run of rows offsets[s] .. offsets[s+1] of
  // expert s, F is [n_slabs,R,C], row i reads X row gather[i] (gather may be null), and the
  // COL product of a slab is complete: col_scale times it goes straight to col_out
  // ([n_slabs,C,R], or [n_slabs,R,C] when col_transposed) instead of col_part.
  const int* offsets;
  const int* gather;
  float* col_out;
  float col_scale;
  int col_transposed;
  int64_t x_rows;     // rows of X (grouped form: bound of the descriptor)
};

// XOR of the 16-byte chunk index of a 256-byte tile row: row-fragment reads (one chunk of
// 16+ consecutive rows) and transposed reads (4 chunks x 4 rows) are both conflict free.
__device__ __forceinline__ int st_swz(int row) { return ((row & 3) << 2) | ((row >> 2) & 3); }

typedef __attribute__((__vector_size__(4 * sizeof(short)))) short st_shortx4;
typedef __attribute__((address_space(3))) st_shortx4* st_lds_shortx4_ptr;

// Transposed fragment of the tile at `tile`: lane (m, h) gets column d0 + m of rows
// k0 + 4h + {0..3} and k0 + 8 + 4h + {0..3}.  The LDS transpose read works on groups of 16
// lanes: lane 4e+g supplies the address of 4 consecutive halfwords, lane i receives, as
// element e, halfword i % 4 of what lane 4e + i / 4 addressed.
__device__ __forceinline__ bf16x8 st_tr_frag(const char* tile, int lane, int k0, int d0) {
  const int b = lane >> 4, i = lane & 15;
  const int col = d0 + 16 * (b & 1) + 4 * (i & 3);
  const int r0 = k0 + 4 * (b >> 1) + (i >> 2), r1 = r0 + 8;
  const st_shortx4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
      (st_lds_shortx4_ptr)(tile + r0 * ST_ROW_BYTES + (((col >> 3) ^ st_swz(r0)) * 16) + (col & 4) * 2));
  const st_shortx4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
      (st_lds_shortx4_ptr)(tile + r1 * ST_ROW_BYTES + (((col >> 3) ^ st_swz(r1)) * 16) + (col & 4) * 2));
  typedef __attribute__((__vector_size__(8 * sizeof(short)))) short shortx8;
  const shortx8 v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  return __builtin_bit_cast(bf16x8, v);
}

// NTE: 32-wide tiles of e (rank <= 32 NTE); NCT: 128-column tiles per chunk; NST: LDS stages.
// All memory traffic of the main loop is LDS DMA, ordered by hand with s_waitcnt vmcnt(n)
// (the compiler inserts no waits for it): per wave, a tile is 8 DMA instructions, the Y rows
// of a row tile R / 8, a flush of the ROW accumulators 4 NTE stores.
// GATHER: the grouped form with a row gather.  The gather indices travel by DMA as well (an
// ordinary global load in the issue path would make the compiler wait for every outstanding
// operation, the ring included): each wave fetches the 32 indices of its own rows of row tile
// q into a private slot, NST row tiles ahead of the first tile that needs them, ordered
// (p % 8) 4 + p / 8 so that a lane reads the 8 it needs as two 16-byte LDS loads.
template <int NTE, int NCT, int NST, bool GATHER>
__device__ __forceinline__ void lora_stats_body(const StatsParams& p, const int block) {
  constexpr int CC = NCT * ST_TILE;
  constexpr int FPITCH = CC + 8;  // halfwords; +16 bytes: rows e land in different banks
  constexpr int YRAW_BYTES = ST_TILE * NTE * 32 * 4;
  // one array for everything the DMA writes: the tile ring, then the Y rows of a row tile ([t][R] f32)
  constexpr int IDX_SLOTS = NST + 1;
  constexpr int IDX_BYTES = GATHER ? 4 * IDX_SLOTS * 256 : 0;
  __shared__ __attribute__((aligned(1024))) char ring[NST * ST_TILE_BYTES + YRAW_BYTES + IDX_BYTES];
  __shared__ __attribute__((aligned(16))) uint16_t fac[NTE * 32 * FPITCH];
  char* const yraw = ring + NST * ST_TILE_BYTES;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int m = lane & 31, half = lane >> 5;
  const int slab = block / p.n_chunks, chunk = block - slab * p.n_chunks;
  const bool grouped = p.offsets != nullptr;
  const int64_t t0 = grouped ? (int64_t)p.offsets[slab] : (int64_t)slab * p.rows_per_slab;
  const int64_t c0 = (int64_t)chunk * p.cc;
  const int rows_here = grouped ? p.offsets[slab + 1] - p.offsets[slab]
                                : (int)(p.T - t0 < p.rows_per_slab ? p.T - t0 : p.rows_per_slab);
  const int n_rt = (rows_here + ST_TILE - 1) / ST_TILE;
  const int cols_here = (int)(p.C - c0 < p.cc ? p.C - c0 : p.cc);
  const int nct = (cols_here + ST_TILE - 1) / ST_TILE;
  const int nt = n_rt * nct;
  const bool do_row = p.F != nullptr, do_col = p.Y != nullptr;
  const int R = p.R;
  const uint16_t* F = grouped && do_row ? p.F + (int64_t)slab * R * p.C : p.F;

  // descriptors at the slab's first row (grouped form: at the first row of X, whose rows are
  // then addressed through the gather or by sorted position); reads past the end return zero
  const int64_t xbase = grouped ? 0 : t0;
  const int64_t left = ((grouped ? p.x_rows : p.T) - xbase) * p.C * 2;
  const dma_rsrc_t rsrc = dma_make_rsrc(p.X + xbase * p.C, (uint32_t)(left < 0x7fffffff ? left : 0x7fffffff));
  // (grouped form: up to the end of the expert's rows, so that the rows of a tile past that end
  // read as zero and add nothing to the COL product)
  const int64_t yleft = do_col ? (grouped ? (int64_t)rows_here : p.T - t0) * R * 4 : 0;
  const dma_rsrc_t yrsrc =
      dma_make_rsrc(do_col ? p.Y + t0 * R : nullptr, (uint32_t)(yleft < 0x7fffffff ? yleft : 0x7fffffff));
  const uint32_t ring_addr = lds_addr_of(ring);
  constexpr int IDX_OFF = NST * ST_TILE_BYTES + YRAW_BYTES;
  const dma_rsrc_t irsrc = dma_make_rsrc(GATHER ? p.gather + t0 : nullptr, GATHER ? (uint32_t)rows_here * 4u : 0u);
  auto issue_idx = [&](int q) {
    const int pp = lane & 31;
    int rg = q * ST_TILE + wave * 32 + (pp & 7) * 4 + (pp >> 3);
    rg = rg < rows_here ? rg : rows_here - 1;
    dma_load4(irsrc, rg * 4, 0, ring_addr + IDX_OFF + (wave * IDX_SLOTS + q % IDX_SLOTS) * 256);
  };
  auto issue_tile = [&](int i) {
    const int rt = i / nct, ct = i - rt * nct;
    const uint32_t stage = ring_addr + (i % NST) * ST_TILE_BYTES;
    int gidx[8];
    if constexpr (GATHER) {
      const int4* ip = (const int4*)(ring + IDX_OFF + (wave * IDX_SLOTS + rt % IDX_SLOTS) * 256 + (lane >> 4) * 32);
      const int4 lo = ip[0], hi = ip[1];
      gidx[0] = lo.x; gidx[1] = lo.y; gidx[2] = lo.z; gidx[3] = lo.w;
      gidx[4] = hi.x; gidx[5] = hi.y; gidx[6] = hi.z; gidx[7] = hi.w;
    }
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const int instr = wave * 8 + k;
      const int row = instr * 4 + (lane >> 4);
      int rg = rt * ST_TILE + row;
      rg = rg < rows_here ? rg : rows_here - 1;
      int64_t xrow = rg;
      if constexpr (GATHER) xrow = gidx[k];
      else if (grouped) xrow = t0 + rg;
      const int c = (lane & 15) ^ st_swz(row);
      // columns past the end of a row (the ragged last column tile) re-read the row's first
      // chunk instead: their ROW factor is zero and their COL results are never stored, and
      // nothing is read outside the row, whatever follows it in memory
      int64_t col = c0 + ct * ST_TILE + c * 8;
      col = col < p.C ? col : 0;
      const int voff = (int)(xrow * p.C * 2) + (int)(col * 2);
      dma_load16(rsrc, voff, 0, stage + instr * 1024);
    }
  };
  // Y rows of row tile rt: 128 R floats, contiguous in memory, land as they are (R / 8 instructions per wave)
  const int ny = R / 8;
  auto issue_y = [&](int rt) {
    for (int k = 0; k < ny; ++k) {
      const int instr = wave * ny + k;
      const int voff = rt * ST_TILE * R * 4 + instr * 1024 + lane * 16;
      dma_load16(yrsrc, voff, 0, ring_addr + NST * ST_TILE_BYTES + instr * 1024);
    }
  };
  if constexpr (GATHER) {
    if (nt > 0) {
#pragma unroll
      for (int q = 0; q < NST; ++q)
        if (q < n_rt) issue_idx(q);
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
  }
  if (do_col && nt > 0) issue_y(0);
#pragma unroll
  for (int i = 0; i < NST - 1; ++i)
    if (i < nt) issue_tile(i);

  // factor of this chunk: fac[e][c] = F[e][c0 + c], zero past R and past C
  if (do_row) {
    for (int i = tid; i < NTE * 32 * (CC / 8); i += 256) {
      const int e = i / (CC / 8), c8 = (i - e * (CC / 8)) * 8;
      uint4 v = make_uint4(0, 0, 0, 0);
      if (e < R && c0 + c8 < p.C) v = *(const uint4*)(F + (int64_t)e * p.C + c0 + c8);
      *(uint4*)(fac + e * FPITCH + c8) = v;
    }
  }

  floatx16 acc_row[NTE];
  floatx16 acc_col[NCT][NTE];
  bf16x8 ya[8][NTE];  // Y^T fragments of the current row tile
#pragma unroll
  for (int et = 0; et < NTE; ++et) {
#pragma unroll
    for (int j = 0; j < 16; ++j) acc_row[et][j] = 0.f;
#pragma unroll
    for (int ct = 0; ct < NCT; ++ct)
#pragma unroll
      for (int j = 0; j < 16; ++j) acc_col[ct][et][j] = 0.f;
  }

  bool stored = false;  // the previous tile ended with a flush (its stores are newer than the DMA before them)
  // One tile; the column tile index is a compile-time constant so that its accumulators are too.
  auto do_tile = [&](int rt, auto ct_tag) {
    constexpr int ct = decltype(ct_tag)::value;
    const int i = rt * nct + ct;
    // tile i has landed (with three stages tile i+1, and the stores of a flush, may still be on their way)
    if (NST == 3 && i + 1 < nt && nct > 1) {
      if (stored) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(8 + 4 * NTE) : "memory");
      else asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
    } else {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    barrier_lds_only();  // ... for every wave, and every wave is done with tile i - 1
    stored = false;
    if (ct == 0 && do_col) {
      // this lane's Y^T fragments: e = 32 et + m, rows 16 ks + 4 half + {0..3} and + 8
      const float* yr = (const float*)yraw;
#pragma unroll
      for (int ks = 0; ks < 8; ++ks)
#pragma unroll
        for (int et = 0; et < NTE; ++et) {
          const int e = 32 * et + m;
          const int ec = e < R ? e : 0;
          bf16x8 v;
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const int t = 16 * ks + 4 * half + (j & 3) + 2 * (j & 4);
            const float y = yr[t * R + ec];
            v[j] = (__bf16)(e < R ? y : 0.f);
          }
          ya[ks][et] = v;
        }
      if (nct == 1) {
        // narrow matrix: the next row tile is the next iteration; fetch its Y rows now
        barrier_lds_only();
        if (rt + 1 < n_rt) issue_y(rt + 1);
      }
    }
    if (ct == 1 && do_col && rt + 1 < n_rt) issue_y(rt + 1);  // yraw is free since this tile's barrier
    if constexpr (GATHER)
      if (ct == 0 && rt + NST < n_rt) issue_idx(rt + NST);  // older than this iteration's tile: landed by the next wait
    if (i + NST - 1 < nt) issue_tile(i + NST - 1);
    const char* tile = ring + (i % NST) * ST_TILE_BYTES;
    if (do_row) {
      const int row = 32 * wave + m;
      const int sw = st_swz(row);
#pragma unroll
      for (int s = 0; s < 8; ++s) {
        const bf16x8 xb = *(const bf16x8*)(tile + row * ST_ROW_BYTES + (((2 * s + half) ^ sw) * 16));
#pragma unroll
        for (int et = 0; et < NTE; ++et) {
          const bf16x8 fa = *(const bf16x8*)(fac + (32 * et + m) * FPITCH + ct * ST_TILE + 16 * s + 8 * half);
          acc_row[et] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa, xb, acc_row[et], 0, 0, 0);
        }
      }
    }
    if (do_col) {
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) {
        const bf16x8 xb = st_tr_frag(tile, lane, 16 * ks, 32 * wave);
#pragma unroll
        for (int et = 0; et < NTE; ++et)
          acc_col[ct][et] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ya[ks][et], xb, acc_col[ct][et], 0, 0, 0);
      }
    }
    if (do_row && ct == nct - 1) {
      // rows 32 wave + m of this row tile: element j of a tile <-> e = 32 et + (j / 4) 8 + 4 half + j % 4
      const int lrow = rt * ST_TILE + 32 * wave + m;
      const int64_t t = t0 + lrow;
#pragma unroll
      for (int et = 0; et < NTE; ++et) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          // every lane stores (the wait above counts 4 NTE stores): out of range goes to a dummy slot
          const int e0 = 32 * et + 8 * q + 4 * half;
          const bool ok = lrow < rows_here && e0 < R;
          float* dst = ok ? p.row_part + ((int64_t)chunk * p.T + t) * R + e0 : p.row_dummy + (tid & 255) * 4;
          *(floatx4*)dst =
              floatx4{acc_row[et][4 * q], acc_row[et][4 * q + 1], acc_row[et][4 * q + 2], acc_row[et][4 * q + 3]};
        }
#pragma unroll
        for (int j = 0; j < 16; ++j) acc_row[et][j] = 0.f;
      }
      stored = true;
    }
  };
  for (int rt = 0; rt < n_rt; ++rt) {
    do_tile(rt, std::integral_constant<int, 0>{});
    if constexpr (NCT > 1) if (nct > 1) do_tile(rt, std::integral_constant<int, 1>{});
    if constexpr (NCT > 2) if (nct > 2) do_tile(rt, std::integral_constant<int, 2>{});
    if constexpr (NCT > 3) if (nct > 3) do_tile(rt, std::integral_constant<int, 3>{});
  }
  if (do_col) {
#pragma unroll
    for (int ct = 0; ct < NCT; ++ct) {
      const int64_t c = c0 + ct * ST_TILE + 32 * wave + m;
      if (ct >= nct || c >= p.C) continue;
#pragma unroll
      for (int et = 0; et < NTE; ++et)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int e0 = 32 * et + 8 * q + 4 * half;
          if (e0 >= R) continue;
          floatx4 v = floatx4{acc_col[ct][et][4 * q], acc_col[ct][et][4 * q + 1], acc_col[ct][et][4 * q + 2],
                              acc_col[ct][et][4 * q + 3]};
          if (!grouped) {
            *(floatx4*)(p.col_part + ((int64_t)slab * p.C + c) * R + e0) = v;
          } else if (!p.col_transposed) {
            *(floatx4*)(p.col_out + ((int64_t)slab * p.C + c) * R + e0) = v * p.col_scale;
          } else {
#pragma unroll
            for (int k = 0; k < 4; ++k) p.col_out[((int64_t)slab * R + e0 + k) * p.C + c] = v[k] * p.col_scale;
          }
        }
    }
  }
}

template <int NTE, int NCT, int NST, bool GATHER>
__global__ __launch_bounds__(256) void lora_stats_kernel(StatsParams p) {
  lora_stats_body<NTE, NCT, NST, GATHER>(p, (int)blockIdx.x);
}

// Several independent passes (the upstream gradients of projections that share an input) in one
// launch: work-groups block0[i] .. block0[i+1]-1 run pass i.
constexpr int STATS_MULTI_MAX = 4;
struct StatsMulti {
  StatsParams p[STATS_MULTI_MAX];
  int block0[STATS_MULTI_MAX + 1];
  int n;
};
template <int NTE, int NCT, int NST>
__global__ __launch_bounds__(256) void lora_stats_multi_kernel(StatsMulti m) {
  int i = 0;
  while (i + 1 < m.n && (int)blockIdx.x >= m.block0[i + 1]) ++i;
  lora_stats_body<NTE, NCT, NST, false>(m.p[i], (int)blockIdx.x - m.block0[i]);
}

// out[i][e] = scale * sum over parts (fixed order) of part[k][i][e]; written as f32 [n][R] (or
// [R][n] when transposed) and, optionally, as bf16 [n][RP] times bf16_scale, zero padded to RP.
struct StatsReduceJob {
  const float* part;
  int n_parts;
  int64_t n;
  float scale;
  float* out;
  int transposed;
  uint16_t* out_bf16;
  int RP;
  float bf16_scale;
  // plain (not transposed) output: row pitch and first column of the R results inside a wider
  // [n][out_ld] array (0: dense [n][R])
  int out_ld = 0, out_off = 0;
  // transposed output split over several arrays: results e_start[i] <= e < e_start[i+1] go to
  // outs[i] as [e - e_start[i]][n] (n_split == 0: everything to `out`)
  int n_split = 0;
  float* outs[4] = {nullptr, nullptr, nullptr, nullptr};
  int e_start[5] = {0, 0, 0, 0, 0};
};

__device__ __forceinline__ void stats_reduce_one(const StatsReduceJob& j, int R, int64_t i) {
  const int width = j.out_bf16 ? j.RP : R;
  if (i >= j.n * width) return;
  const int64_t row = i / width;
  const int e = (int)(i - row * width);
  float s = 0.f;
  if (e < R) {
    const int64_t stride = j.n * R;
    const float* src = j.part + row * R + e;
    // eight loads in flight per thread; the order of the additions is fixed
    for (int k0 = 0; k0 < j.n_parts; k0 += 8) {
      float v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = k0 + u < j.n_parts ? src[(k0 + u) * stride] : 0.f;
#pragma unroll
      for (int u = 0; u < 8; ++u) s += v[u];
    }
    s *= j.scale;
    if (j.transposed) {
      if (j.n_split > 0) {
        // (constant indices only: a run-time index into the job would send it through scratch memory)
        float* dst = j.outs[0];
        int e0 = 0;
#pragma unroll
        for (int k = 1; k < 4; ++k)
          if (k < j.n_split && e >= j.e_start[k]) {
            dst = j.outs[k];
            e0 = j.e_start[k];
          }
        dst[(int64_t)(e - e0) * j.n + row] = s;
      } else {
        j.out[(int64_t)e * j.n + row] = s;
      }
    } else {
      j.out[row * (j.out_ld ? j.out_ld : R) + j.out_off + e] = s;
    }
  }
  if (j.out_bf16) j.out_bf16[row * j.RP + e] = f32_to_bf16(s * j.bf16_scale);
}

__global__ __launch_bounds__(256) static void stats_reduce_kernel(StatsReduceJob a, StatsReduceJob b, int R, int nblk_a) {
  // (each job is used where it lies, among the kernel arguments: a selected copy would live in scratch memory)
  if ((int)blockIdx.x < nblk_a) stats_reduce_one(a, R, (int64_t)blockIdx.x * 256 + threadIdx.x);
  else stats_reduce_one(b, R, (int64_t)(blockIdx.x - nblk_a) * 256 + threadIdx.x);
}

struct StatsGeom {
  int cc, rows_per_slab, n_slabs, n_chunks;
};
static inline int stats_num_cus() {
  int cus = 0, dev = 0;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
    cus = 256;
  return cus;
}
// Chunk width by rank (the factor and the accumulators of a chunk live in LDS / registers);
// slab height so that the grid is one round of work-groups (one fits per CU) when the matrix
// is large enough: a second, partly filled round would cost as much as the first.
// Cost of a grid in half tile times: rounds of work-groups on the CUs, each as long as its tiles
// (a row tile of cct column tiles also writes its ROW partial, about half a tile time) plus
// about two tile times of set-up (factor load, filling the ring, flushing the accumulators).
static inline int64_t stats_grid_cost(int64_t blocks, int64_t row_tiles_per_block, int cct) {
  const int64_t cus = stats_num_cus();
  return ((blocks + cus - 1) / cus) * (row_tiles_per_block * (2 * cct + 1) + 4);
}

static inline StatsGeom stats_geom(int64_t T, int64_t C, int r) {
  const int max_cct = r > 32 ? 2 : 4;  // column tiles per chunk the kernel holds accumulators for
  const int64_t row_tiles = (T + ST_TILE - 1) / ST_TILE, col_tiles = (C + ST_TILE - 1) / ST_TILE;
  // row offsets inside a slab are 31-bit byte offsets
  const int64_t cap = ((1ll << 31) - 1) / (2 * C) / ST_TILE;
  StatsGeom best{};
  int64_t best_cost = -1;
  for (int cct = max_cct; cct >= 1; --cct) {
    const int64_t n_chunks = (col_tiles + cct - 1) / cct;
    int64_t want = stats_num_cus() / n_chunks;
    want = want < 1 ? 1 : (want > row_tiles ? row_tiles : want);
    for (int64_t w = want; w <= want + 1 && w <= row_tiles; ++w) {
      int64_t slab_tiles = (row_tiles + w - 1) / w;
      if (slab_tiles > cap) slab_tiles = cap < 1 ? 1 : cap;
      const int64_t n_slabs = (row_tiles + slab_tiles - 1) / slab_tiles;
      const int64_t cost = stats_grid_cost(n_slabs * n_chunks, slab_tiles, cct);
      if (best_cost < 0 || cost < best_cost) {
        best_cost = cost;
        best.cc = cct * ST_TILE;
        best.n_chunks = (int)n_chunks;
        best.rows_per_slab = (int)(slab_tiles * ST_TILE);
        best.n_slabs = (int)n_slabs;
      }
    }
  }
  return best;
}

static inline StatsParams stats_params(const void* X, int64_t T, int64_t C, const uint16_t* F, const float* Y, int r,
                                       const StatsGeom& g, float* row_part, float* col_part, float* row_dummy) {
  StatsParams p;
  p.X = (const uint16_t*)X;
  p.T = T;
  p.C = C;
  p.F = F;
  p.Y = Y;
  p.row_part = row_part;
  p.col_part = col_part;
  p.row_dummy = row_dummy;
  p.offsets = nullptr;
  p.gather = nullptr;
  p.col_out = nullptr;
  p.col_scale = 0.f;
  p.col_transposed = 0;
  p.x_rows = T;
  p.R = r;
  p.rows_per_slab = g.rows_per_slab;
  p.n_slabs = g.n_slabs;
  p.n_chunks = g.n_chunks;
  p.cc = g.cc;
  return p;
}

static inline int32_t launch_stats(const void* X, int64_t T, int64_t C, const uint16_t* F, const float* Y, int r,
                            const StatsGeom& g, float* row_part, float* col_part, float* row_dummy,
                            hipStream_t st) {
  const StatsParams p = stats_params(X, T, C, F, Y, r, g, row_part, col_part, row_dummy);
  const unsigned grid = (unsigned)(g.n_slabs * g.n_chunks);
  if (r > 32)
    lora_stats_kernel<2, 2, 2, false><<<grid, 256, 0, st>>>(p);
  else
    lora_stats_kernel<1, 4, 3, false><<<grid, 256, 0, st>>>(p);
  ARTK_CHECK_LAUNCH();
  return ARTK_OK;
}

// The passes of m in one launch; all ranks on the same side of 32 (the caller checks).
static inline int32_t launch_stats_multi(StatsMulti& m, bool wide_rank, hipStream_t st) {
  int blocks = 0;
  for (int i = 0; i < m.n; ++i) {
    m.block0[i] = blocks;
    blocks += m.p[i].n_slabs * m.p[i].n_chunks;
  }
  m.block0[m.n] = blocks;
  if (wide_rank)
    lora_stats_multi_kernel<2, 2, 2><<<(unsigned)blocks, 256, 0, st>>>(m);
  else
    lora_stats_multi_kernel<1, 4, 3><<<(unsigned)blocks, 256, 0, st>>>(m);
  ARTK_CHECK_LAUNCH();
  return ARTK_OK;
}


// Grouped form: slab = expert.  ROW partials go to row_part [n_chunks][n_rows][r]; the COL
// product of each expert is written to col_out, scaled.
static inline int stats_grouped_cc(int64_t C, int r, int E) {
  const int max_cct = r > 32 ? 2 : 4;
  const int64_t col_tiles = (C + ST_TILE - 1) / ST_TILE;
  int best = max_cct;
  int64_t best_cost = -1;
  for (int cct = max_cct; cct >= 1; --cct) {
    const int64_t n_chunks = (col_tiles + cct - 1) / cct;
    const int64_t cost = stats_grid_cost((int64_t)E * n_chunks, 2, cct);  // a couple of row tiles per expert
    if (best_cost < 0 || cost < best_cost) {
      best_cost = cost;
      best = cct;
    }
  }
  return best * ST_TILE;
}
static inline int stats_grouped_chunks(int64_t C, int r, int E) {
  const int cc = stats_grouped_cc(C, r, E);
  return (int)((C + cc - 1) / cc);
}
static inline int32_t launch_stats_grouped(const void* X, int64_t x_rows, const int* gather, int64_t n_rows,
                                           int64_t C, const uint16_t* F, const float* Y, int r, int E,
                                           const int* offsets, float* row_part, float* col_out,
                                           float col_scale, int col_transposed, float* row_dummy,
                                           hipStream_t st) {
  StatsParams p;
  p.X = (const uint16_t*)X;
  p.T = n_rows;
  p.C = C;
  p.F = F;
  p.Y = Y;
  p.row_part = row_part;
  p.col_part = nullptr;
  p.row_dummy = row_dummy;
  p.offsets = offsets;
  p.gather = gather;
  p.col_out = col_out;
  p.col_scale = col_scale;
  p.col_transposed = col_transposed;
  p.x_rows = x_rows;
  p.R = r;
  p.rows_per_slab = 0;
  p.n_slabs = E;
  p.cc = stats_grouped_cc(C, r, E);
  p.n_chunks = stats_grouped_chunks(C, r, E);
  const unsigned grid = (unsigned)(E * p.n_chunks);
  if (gather) {
    if (r > 32)
      lora_stats_kernel<2, 2, 2, true><<<grid, 256, 0, st>>>(p);
    else
      lora_stats_kernel<1, 4, 3, true><<<grid, 256, 0, st>>>(p);
  } else {
    if (r > 32)
      lora_stats_kernel<2, 2, 2, false><<<grid, 256, 0, st>>>(p);
    else
      lora_stats_kernel<1, 4, 3, false><<<grid, 256, 0, st>>>(p);
  }
  ARTK_CHECK_LAUNCH();
  return ARTK_OK;
}

static inline int32_t launch_stats_reduce(const StatsReduceJob& a, const StatsReduceJob& b, int r, hipStream_t st) {
  const int64_t na = a.n * (a.out_bf16 ? a.RP : r), nb = b.n * (b.out_bf16 ? b.RP : r);
  const int blk_a = (int)((na + 255) / 256), blk_b = (int)((nb + 255) / 256);
  stats_reduce_kernel<<<(unsigned)(blk_a + blk_b), 256, 0, st>>>(a, b, r, blk_a);
  ARTK_CHECK_LAUNCH();
  return ARTK_OK;
}

// Up to 2 * STATS_MULTI_MAX reductions in one launch; job i reduces partials of rank R[i].
struct StatsReduceMulti {
  StatsReduceJob job[2 * STATS_MULTI_MAX];
  int R[2 * STATS_MULTI_MAX];
  int block0[2 * STATS_MULTI_MAX + 1];
  int n;
};
__global__ __launch_bounds__(256) static void stats_reduce_multi_kernel(StatsReduceMulti m) {
  int k = 0;
  while (k + 1 < m.n && (int)blockIdx.x >= m.block0[k + 1]) ++k;
  stats_reduce_one(m.job[k], m.R[k], (int64_t)((int)blockIdx.x - m.block0[k]) * 256 + threadIdx.x);
}
static inline int32_t launch_stats_reduce_multi(StatsReduceMulti& m, hipStream_t st) {
  int blocks = 0;
  for (int i = 0; i < m.n; ++i) {
    const StatsReduceJob& j = m.job[i];
    m.block0[i] = blocks;
    blocks += (int)((j.n * (j.out_bf16 ? j.RP : m.R[i]) + 255) / 256);
  }
  m.block0[m.n] = blocks;
  stats_reduce_multi_kernel<<<(unsigned)blocks, 256, 0, st>>>(m);
  ARTK_CHECK_LAUNCH();
  return ARTK_OK;
}


}  // namespace artk
