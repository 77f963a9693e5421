// Many small populations at once: one workgroup per population, everything in LDS.
//
// This is the batched form of the same path (what the reference reaches through vmap:
// src/evox/operators/selection/non_dominate.py:107-125 for the peeling, :198-254 under vmap for
// the rest).  Per population the result is identical to the single-population kernels.
//
// Thread j owns row j of its population (blockDim.x = rows rounded up to 64, at most 1024).
//   * dominance: lane = dominated row j, loop over dominators i whose fitness comes from scalar loads
//     (wave-uniform address), `<=` and `<` per objective exactly as non_dominate.py:20-24, masks
//     combined on the scalar unit and shifted into the lane's word with v_addc_co_u32; the 64-bit
//     words of row j go to LDS (row stride W + 1 words against bank conflicts);
//   * counts = popcount of the row; peeling = count -= popcount(row & front) with the front bitmap in
//     LDS and two block barriers per pass; fronts are listed in ascending row order as they appear;
//   * crowding distance and the index-stable top-k on the last front by counting ranks over LDS tiles;
//   * the selected rows are gathered by the whole block.
#pragma once

#include "common.hpp"
#include "dominance.hpp"

// Hook for timing builds (a tool defines it to store a time stamp per workgroup and phase); nothing otherwise.
#ifndef EVX_BATCH_TRACE
#define EVX_BATCH_TRACE(slot)
#endif

namespace evx {

constexpr int kBatchedMaxRows = 1024;
constexpr int kBatchedMaxObjectives = 16;

typedef const float __attribute__((address_space(4))) * ConstFloatPtr;

struct BatchedArgs {
  const float* f;          // (batch, n, m) with strides in elements
  int64_t f_stride_b, f_stride_row, f_stride_col;
  int n, m;
  int stop_count;          // rows to rank before stopping (n = rank everything)
  int* rank_all;           // (batch, n) ranks of all rows, or null
  // selection outputs (all null in rank-only mode)
  const uint8_t* x;        // (batch, n, row_bytes) raw rows, or null
  int64_t x_stride_b, x_row_stride, x_row_bytes;
  int x_unit;              // 16, 4 or 1: copy granularity that pointers, strides and row size allow
  // A population given as two tensors with the same strides (parents and offspring): rows from n_first on are read
  // f_second elements (x: x_second bytes) further on, which is where the second tensor's row 0 lies from row n_first
  // of the first.  One tensor: all zero.
  int n_first;
  int64_t f_second, x_second;
  uint8_t* out_x;          // (batch, topk, row_bytes)
  float* out_f;            // (batch, topk, m)
  int* out_rank;           // (batch, topk)
  float* out_dist;         // (batch, topk)
  // 1: the launch has batched_stage_bytes(nt, m) more dynamic LDS, behind the layout below, and the dominators of the
  // arithmetic test are read from a copy of the fitness there (few small populations: a wave that has its SIMD to
  // itself waits out every scalar load in full, 0.35 us per eight dominators; reads from LDS return in order and are
  // issued ahead); 0: from memory by scalar loads, which is faster once waves share a SIMD -- the LDS has one port
  int stage_fitness;
};

// Number of elements of `tile` (nv entries, (key << 32 | index) pairs) that are smaller than `mine`.
__device__ inline int count_smaller(const uint64_t* tile, int nv, uint64_t mine) {
  int smaller = 0;
  const int lim = (nv + 3) & ~3;  // the tile is padded with all-ones up to a multiple of 4
  for (int e = 0; e < lim; e += 4) {
    const ulonglong2 a = *reinterpret_cast<const ulonglong2*>(tile + e);
    const ulonglong2 b = *reinterpret_cast<const ulonglong2*>(tile + e + 2);
    smaller += (a.x < mine) + (a.y < mine) + (b.x < mine) + (b.y < mine);
  }
  return smaller;
}

// Row stride of the LDS matrix in words: one word of padding against bank conflicts, except at the
// largest size, where the padding would not fit; at least nine words (thirteen above eight objectives),
// because after the peeling the matrix's LDS is reused for everything that the rest of the kernel needs
// (4 bytes per objective, rounded up to eight objectives, plus 28 bytes per row).
__host__ __device__ inline int batched_row_stride(int nt, int m) {
  const int least = m <= 8 ? 9 : 13;
  return nt == 1024 ? 16 : (nt / 64 + 1 < least ? least : nt / 64 + 1);
}

// Dynamic LDS layout (nt = blockDim.x, M8 = the objectives rounded up to a multiple of eight):
//   uint64 dom[nt][row stride] | uint64 front[2][16] | int perm[nt]
// and, once the peeling is over, inside dom:
//   float fit[M8][nt] | uint64 tile[nt + 4] | float scost[nt] | float dist[nt] | int order[nt] | int rank[nt] | int below[nt]
// 512 rows of up to eight objectives take 39.2 KB, so that four workgroups share a compute unit's 160 KB.
__host__ __device__ inline size_t batched_lds_bytes(int nt, int m) {
  return sizeof(uint64_t) * ((size_t)nt * batched_row_stride(nt, m) + 32) + sizeof(int) * (size_t)nt;
}
// The copy of the fitness for BatchedArgs::stage_fitness: rows of the objectives rounded up to a multiple of four.
__host__ __device__ inline int batched_stage_stride(int m) { return (m + 3) & ~3; }
__host__ __device__ inline size_t batched_stage_bytes(int nt, int m) { return sizeof(float) * (size_t)nt * batched_stage_stride(m); }

// Position of every candidate among the nv (key << 32 | index) pairs of `tile`, by counting the smaller
// ones; the count of candidate q is split over `parts` threads (q + nvq * part, nvq = nv rounded up to whole
// waves), which add their shares in `below`.  Every thread of the block calls it; returns the position
// for threads below nv.  tile must be padded with all-ones up to a multiple of 4 entries.
__device__ inline int position_by_counting(const uint64_t* tile, int* below, int nv, int j, int nt) {
  const int nvq = (nv + 63) & ~63;
  const int parts = nt / nvq;  // >= 1: nv <= n <= nt
  if (parts == 1) {
    __syncthreads();
    return j < nv ? count_smaller(tile, nv, tile[j]) : 0;
  }
  if (j < nv) below[j] = 0;
  __syncthreads();
  const int part = j / nvq, q = j - part * nvq;
  if (part < parts && q < nv) {
    const int chunk = (((nv + parts - 1) / parts) + 3) & ~3;
    const int e0 = part * chunk;
    const int e1 = min(e0 + chunk, (nv + 3) & ~3);
    const uint64_t mine = tile[q];
    int smaller = 0;
    for (int e = e0; e < e1; e += 4) {
      const ulonglong2 u = *reinterpret_cast<const ulonglong2*>(tile + e);
      const ulonglong2 v = *reinterpret_cast<const ulonglong2*>(tile + e + 2);
      smaller += (u.x < mine) + (u.y < mine) + (v.x < mine) + (v.y < mine);
    }
    if (smaller) atomicAdd(&below[q], smaller);
  }
  __syncthreads();
  return j < nv ? below[j] : 0;
}

// The selected rows of x as one flat array of units of type T (4 or 16 bytes): unit e of the output is unit
// e % row_units of input row order[e / row_units].  Four units per thread are in flight: a load that waits
// for the store before it costs a memory round trip per unit.
template <class T, class Index>
__device__ inline void gather_units(const uint8_t* __restrict__ xb, uint8_t* __restrict__ dst, const Index* order,
                                    int64_t x_row_stride, uint32_t row_units, uint32_t total, int j, int nt,
                                    int n_first, int64_t x_second) {
  auto row_at = [&](uint32_t p) {
    const int src = order[p];
    return xb + (int64_t)src * x_row_stride + (src >= n_first ? x_second : 0);
  };
  for (uint32_t e = j; e < total; e += 4u * nt) {
    const uint32_t e1 = e + nt, e2 = e + 2u * nt, e3 = e + 3u * nt;
    const uint32_t c0 = e, c1 = e1 < total ? e1 : e, c2 = e2 < total ? e2 : e, c3 = e3 < total ? e3 : e;
    const uint32_t p0 = c0 / row_units, p1 = c1 / row_units, p2 = c2 / row_units, p3 = c3 / row_units;
    const T v0 = *reinterpret_cast<const T*>(row_at(p0) + (int64_t)(c0 - p0 * row_units) * sizeof(T));
    const T v1 = *reinterpret_cast<const T*>(row_at(p1) + (int64_t)(c1 - p1 * row_units) * sizeof(T));
    const T v2 = *reinterpret_cast<const T*>(row_at(p2) + (int64_t)(c2 - p2 * row_units) * sizeof(T));
    const T v3 = *reinterpret_cast<const T*>(row_at(p3) + (int64_t)(c3 - p3 * row_units) * sizeof(T));
    *reinterpret_cast<T*>(dst + (int64_t)c0 * sizeof(T)) = v0;
    if (e1 < total) *reinterpret_cast<T*>(dst + (int64_t)e1 * sizeof(T)) = v1;
    if (e2 < total) *reinterpret_cast<T*>(dst + (int64_t)e2 * sizeof(T)) = v2;
    if (e3 < total) *reinterpret_cast<T*>(dst + (int64_t)e3 * sizeof(T)) = v3;
  }
}

// Registers are capped for eight waves per SIMD (at most 64 VGPRs and 96 SGPRs): populations of 512 rows
// then run four workgroups to a compute unit, which their LDS allows (three above eight objectives).
template <int M>
__global__ __launch_bounds__(1024) __attribute__((amdgpu_waves_per_eu(M <= 12 ? 8 : 4, 8))) void batched_kernel(BatchedArgs a) {
  extern __shared__ uint64_t lds64[];
  const int nt = blockDim.x;
  const int W = nt >> 6;
  const int rs = batched_row_stride(nt, M);
  uint64_t* dom = lds64;
  uint64_t* front = dom + (size_t)nt * rs;
  int* perm = reinterpret_cast<int*>(front + 32);
  // valid only after the peeling (they lie inside dom)
  float* fit_lds = reinterpret_cast<float*>(dom);
  uint64_t* tile = reinterpret_cast<uint64_t*>(fit_lds + ((M + 7) / 8 * 8) * (size_t)nt);
  float* scost = reinterpret_cast<float*>(tile + (nt + 4));
  float* dist = scost + nt;
  int* order = reinterpret_cast<int*>(dist + nt);
  int* rank_lds = order + nt;
  int* below = rank_lds + nt;

  const int n = a.n;
  const int j = threadIdx.x;
  const int lane = j & 63;
  const int wave = j >> 6;
  const bool valid = j < n;
  const float* __restrict__ f = a.f + (int64_t)blockIdx.x * a.f_stride_b;
  const float nan = __uint_as_float(0x7FC00000u);

  EVX_BATCH_TRACE(0);
  float xj[M];
#pragma unroll
  for (int k = 0; k < M; ++k)
    xj[k] = valid ? f[(int64_t)j * a.f_stride_row + k * a.f_stride_col + (j >= a.n_first ? a.f_second : 0)] : nan;

  // ---- dominance: word w of row j = which rows 64 w .. 64 w + 63 dominate row j.  When every value of
  // the population is finite the test is the arithmetic one of dominance.hpp (signs of the differences
  // x[j,k] - x[i,k]; the lane's own values with -0.0 turned into +0.0, which is all that form needs).
  bool finite_row = true;
  float xz[M];
#pragma unroll
  for (int k = 0; k < M; ++k) {
    finite_row &= !valid || fabsf(xj[k]) <= 3.4028234663852886e38f;
    xz[k] = xj[k] + 0.0f;
  }
  constexpr int MS = (M + 3) & ~3;
  // (behind the layout above, 16-byte aligned; the address is formed where it is used: one register less to keep)
  auto stage_of = [&]() { return reinterpret_cast<float*>(reinterpret_cast<uint8_t*>(lds64) + batched_lds_bytes(nt, M)); };
  constexpr bool kMayStage = M <= 8;  // (with more objectives the extra path costs the kernel a register it does not have)
  if (kMayStage && a.stage_fitness) {
    float* const stage = stage_of();
#pragma unroll
    for (int k = 0; k < M; ++k) stage[j * MS + k] = xj[k];
  }
  const bool all_finite = __syncthreads_and(finite_row) != 0;
  const bool packed_rows = a.f_stride_col == 1 && a.f_stride_row == M;
  constexpr int GP = M <= 8 ? 8 : 4;  // dominators per group of scalar loads (at most 64 scalars)
  // Dominators are read at wave-uniform addresses through the constant address space: the fitness is never
  // written here, and only loads known to be invariant are issued as scalar loads.
  const ConstFloatPtr fc = (ConstFloatPtr)f;
  int cnt = 0;
  for (int w = 0; w < W; ++w) {
    uint32_t half[2];
#pragma unroll
    for (int h = 1; h >= 0; --h) {
      uint32_t acc = 0;
      const int i0 = w * 64 + h * 32;
      const int64_t second0 = i0 >= a.n_first ? a.f_second : 0;
      if (kMayStage && all_finite && a.stage_fitness) {
        // (rows from n on hold NaN: a lane's test against them is discarded)
#pragma unroll 8
        for (int t = 31; t >= 0; --t) {
          const int i = i0 + t;  // wave-uniform
          float v[MS];
#pragma unroll
          for (int q = 0; q < MS / 4; ++q) {
            const float4 piece = *reinterpret_cast<const float4*>(stage_of() + i * MS + 4 * q);
            v[4 * q] = piece.x; v[4 * q + 1] = piece.y; v[4 * q + 2] = piece.z; v[4 * q + 3] = piece.w;
          }
          uint32_t o = 0u;
#pragma unroll
          for (int k = 0; k < M; ++k) o |= __float_as_uint(xz[k] - v[k]);
          acc = shift_in_positive(acc, i < n ? o : 0u);
        }
      } else if (all_finite && packed_rows && i0 + 32 <= n && (i0 + 32 <= a.n_first || i0 >= a.n_first)) {
        // rows of M consecutive floats: GP dominators are GP M consecutive scalars, fetched by wide scalar loads
        // (the 32 dominators come from one tensor)
#pragma unroll 1
        for (int g = 32 / GP - 1; g >= 0; --g) {
          const ConstFloatPtr p = fc + (int64_t)(i0 + g * GP) * M + second0;  // wave-uniform
          float v[GP * M];
#pragma unroll
          for (int e = 0; e < GP * M; ++e) v[e] = p[e];
#pragma unroll
          for (int u = GP - 1; u >= 0; --u) {
            uint32_t o = 0u;
#pragma unroll
            for (int k = 0; k < M; ++k) o |= __float_as_uint(xz[k] - v[u * M + k]);
            acc = shift_in_positive(acc, o);
          }
        }
      } else if (all_finite) {
#pragma unroll 8
        for (int t = 31; t >= 0; --t) {
          const int i = w * 64 + h * 32 + t;  // wave-uniform
          const int ic = i < n ? i : 0;
          uint32_t o = 0u;
#pragma unroll
          for (int k = 0; k < M; ++k)
            o |= __float_as_uint(xz[k] - fc[(int64_t)ic * a.f_stride_row + k * a.f_stride_col + (ic >= a.n_first ? a.f_second : 0)]);
          acc = shift_in_positive(acc, i < n ? o : 0u);
        }
      } else {
#pragma unroll 8
        for (int t = 31; t >= 0; --t) {
          const int i = w * 64 + h * 32 + t;  // wave-uniform
          const int ic = i < n ? i : 0;
          uint64_t le = i < n ? ~0ull : 0ull;
          uint64_t lt = 0ull;
#pragma unroll
          for (int k = 0; k < M; ++k) {
            const float xi = fc[(int64_t)ic * a.f_stride_row + k * a.f_stride_col + (ic >= a.n_first ? a.f_second : 0)];
            le &= __builtin_amdgcn_ballot_w64(xi <= xj[k]);
            lt |= __builtin_amdgcn_ballot_w64(xi < xj[k]);
          }
          acc = shift_in(acc, le & lt);
        }
      }
      half[h] = acc;
    }
    const uint64_t word = valid ? (((uint64_t)half[1] << 32) | half[0]) : 0ull;
    dom[(size_t)j * rs + w] = word;
    cnt += __popcll(word);
  }

  EVX_BATCH_TRACE(1);
  // ---- peeling (non_dominate.py:29-59, :107-125), fronts listed in ascending row order
  int rank = valid ? kRankUnset : -1;
  int level = 0, ranked = 0;
  int worst_start = 0, nv = 0;
  {
    const uint64_t b = __builtin_amdgcn_ballot_w64(valid && cnt == 0);
    if (lane == 0) front[wave] = b;
    if (valid && cnt == 0) rank = 0;
  }
  for (;;) {
    __syncthreads();
    const uint64_t* cur = front + (level & 1) * 16;
    uint64_t* nxt = front + ((level + 1) & 1) * 16;
    int size = 0, before = 0;
    for (int w = 0; w < W; ++w) {
      const int c = __popcll(cur[w]);
      size += c;
      if (w < wave) before += c;
    }
    if (rank == level) perm[ranked + before + __popcll(cur[wave] & ((1ull << lane) - 1ull))] = j;
    if (size == 0 || ranked + size >= a.stop_count) {
      worst_start = ranked;
      nv = size;
      break;
    }
    bool newly = false;
    if (rank == kRankUnset) {
      int c = 0;
      for (int w = 0; w < W; ++w) c += __popcll(dom[(size_t)j * rs + w] & cur[w]);
      cnt -= c;
      newly = cnt == 0;
      if (newly) rank = level + 1;
    }
    const uint64_t b = __builtin_amdgcn_ballot_w64(newly);
    if (lane == 0) nxt[wave] = b;
    ranked += size;
    ++level;
  }
  if (a.rank_all && valid) a.rank_all[(int64_t)blockIdx.x * n + j] = rank;
  if (a.out_f == nullptr) return;  // rank-only mode

  EVX_BATCH_TRACE(2);
  // ---- crowding distance of the last front (non_dominate.py:198-231 with mask = rank == worst)
  // Every thread is past its last read of the matrix (the loop above leaves after a barrier): its LDS now
  // holds the fitness by objective (fit_lds[k * nt + row]) and the arrays of the steps below, so that
  // candidates and the final gather read other rows' values from LDS instead of from memory again.
  const int topk = a.stop_count;
  const int need = topk - worst_start;
  rank_lds[j] = rank;
  dist[j] = -INFINITY;
#pragma unroll
  for (int k = 0; k < M; ++k) fit_lds[k * nt + j] = xj[k];
  __syncthreads();
  const bool cand = j < nv;                      // thread q = candidate q of the last front
  const int row = cand ? perm[worst_start + j] : 0;
  bool boundary = false;
  float acc = 0.0f;
#pragma unroll
  for (int k = 0; k < M; ++k) {
    const float cost = cand ? fit_lds[k * nt + row] : 0.0f;
    if (j < nv + 4) tile[j] = cand ? ((uint64_t)ordered_key(cost) << 32) | (uint32_t)j : ~0ull;
    if (j < 4 && nv + j >= nt) tile[nv + j] = ~0ull;  // padding past the thread count
    const int p = position_by_counting(tile, below, nv, j, nt);
    if (cand) scost[p] = cost;
    __syncthreads();
    if (cand) {
      if (p == 0 || p == nv - 1) {
        boundary = true;
      } else {
        const float term = (scost[p + 1] - scost[p - 1]) / (scost[nv - 1] - scost[0]);
        acc = k == 0 ? term : acc + term;
      }
    }
    // (the barriers inside the next position_by_counting separate these reads from the next writes of scost)
  }
  const float d = boundary ? INFINITY : acc;
  if (cand) dist[row] = d;

  EVX_BATCH_TRACE(3);
  // ---- index-stable top-k on the last front by (-distance, row index) (non_dominate.py:253)
  {
    if (j < nv + 4) tile[j] = cand ? ((uint64_t)ordered_key(-d) << 32) | (uint32_t)j : ~0ull;
    if (j < 4 && nv + j >= nt) tile[nv + j] = ~0ull;
    const int p = position_by_counting(tile, below, nv, j, nt);
    if (cand && p < need) order[worst_start + p] = row;
    if (j < worst_start) order[j] = perm[j];
  }
  __syncthreads();

  EVX_BATCH_TRACE(4);
  // ---- gather the topk selected rows
  const int64_t ob = (int64_t)blockIdx.x * topk;
  for (int p = j; p < topk; p += nt) {
    const int src = order[p];
    a.out_rank[ob + p] = rank_lds[src];
    a.out_dist[ob + p] = dist[src];
#pragma unroll
    for (int k = 0; k < M; ++k) a.out_f[(ob + p) * M + k] = fit_lds[k * nt + src];
  }
  if (a.x != nullptr) {
    const uint8_t* __restrict__ xb = a.x + (int64_t)blockIdx.x * a.x_stride_b;
    uint8_t* __restrict__ dst = a.out_x + ob * a.x_row_bytes;
    const int64_t row_units = a.x_row_bytes / a.x_unit;
    const int64_t total = row_units * topk;
    if (a.x_unit >= 4 && total < (1ll << 31)) {
      if (a.x_unit == 16)
        gather_units<uint4>(xb, dst, order, a.x_row_stride, (uint32_t)row_units, (uint32_t)total, j, nt, a.n_first, a.x_second);
      else
        gather_units<uint32_t>(xb, dst, order, a.x_row_stride, (uint32_t)row_units, (uint32_t)total, j, nt, a.n_first, a.x_second);
    } else {
      const int waves = nt >> 6;
      for (int p = wave; p < topk; p += waves) {
        const uint8_t* __restrict__ sp = xb + (int64_t)order[p] * a.x_row_stride + (order[p] >= a.n_first ? a.x_second : 0);
        uint8_t* __restrict__ dp = dst + (int64_t)p * a.x_row_bytes;
        if (a.x_unit == 16) {
          for (int64_t b = lane * 16; b < a.x_row_bytes; b += 64 * 16)
            *reinterpret_cast<uint4*>(dp + b) = *reinterpret_cast<const uint4*>(sp + b);
        } else if (a.x_unit == 4) {
          for (int64_t b = lane * 4; b < a.x_row_bytes; b += 64 * 4)
            *reinterpret_cast<uint32_t*>(dp + b) = *reinterpret_cast<const uint32_t*>(sp + b);
        } else {
          for (int64_t b = lane; b < a.x_row_bytes; b += 64) dp[b] = sp[b];
        }
      }
    }
  }
  EVX_BATCH_TRACE(5);
}

}  // namespace evx
