// Building blocks of the crowding distance and the selection: mask compaction, ranking by counting,
// the distance formula, the fused row gather and the tournament pick (the kernels that order the last
// front are in finish.hpp).
//
// Reference semantics:
//   crowding_distance            src/evox/operators/selection/non_dominate.py:198-231
//   lexsort (stable, last key primary)   src/evox/utils/jit_fix_operator.py:246-252
//   nd_environmental_selection   non_dominate.py:234-254
//
// The candidate list L (ascending row index, nv entries) is either the last front as listed by the
// peel kernel or the compacted mask.  Per objective k the candidates are ordered by
// (ordered_key(cost), position in L): that is torch's stable ascending sort with NaN last and signed
// zeros tied, restricted to the masked rows, which the reference puts first (non_dominate.py:215-221).
// The ordering is computed as a rank by counting, pos(q) = #{q' : (key', q') < (key, q)}: every
// candidate is compared with every other one, the partners streaming through LDS in tiles.  The
// counts give the sorted position directly, with no passes that depend on one another.
#pragma once

#include "common.hpp"

namespace evx {

// Stable compaction of a boolean mask into an ascending list (one block; n is at most a few 10^5).
// mask == nullptr selects every row.  Also fills dist with -inf and publishes nv in ctrl.
// (Several populations in the launch, one per blockIdx.z: their masks lie mask_step bytes apart.)
__global__ __launch_bounds__(1024) void compact_mask_kernel(const uint8_t* __restrict__ mask, int64_t mask_stride, int n,
                                                            int* __restrict__ list, float* __restrict__ dist,
                                                            Ctrl* __restrict__ ctrl, int64_t mask_step, int64_t ws_step) {
  if (mask != nullptr) mask += (int64_t)blockIdx.z * mask_step;
  to_population(ws_step, list, dist, ctrl);
  // A wave takes a run of consecutive rows, 64 at a time: it counts its selected rows (loads that depend on nothing:
  // several in flight), the runs' counts are added up once, and a second walk writes the list.  (One step of 1024
  // rows at a time with the running total handed on through LDS cost three barriers and a memory round trip per
  // step: 21 us for 20 000 rows.)
  __shared__ int wave_tot[16];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int waves = blockDim.x >> 6;
  const int per_wave = ((n + waves - 1) / waves + 63) & ~63;
  const int r0 = wave * per_wave, r1 = min(n, r0 + per_wave);
  auto selected = [&](int j) { return j < r1 && (mask == nullptr || mask[(int64_t)j * mask_stride] != 0); };
  int count = 0;
#pragma unroll 4
  for (int j0 = r0; j0 < r1; j0 += 64) {
    const int j = j0 + lane;
    if (j < r1) dist[j] = -INFINITY;
    count += __popcll(__builtin_amdgcn_ballot_w64(selected(j)));
  }
  if (lane == 0) wave_tot[wave] = count;
  __syncthreads();
  int offset = 0, total = 0;
  for (int w = 0; w < waves; ++w) {
    if (w < wave) offset += wave_tot[w];
    total += wave_tot[w];
  }
#pragma unroll 4
  for (int j0 = r0; j0 < r1; j0 += 64) {
    const int j = j0 + lane;
    const bool on = selected(j);
    const uint64_t b = __builtin_amdgcn_ballot_w64(on);
    if (on) list[offset + __popcll(b & ((1ull << lane) - 1ull))] = j;
    offset += __popcll(b);
  }
  if (threadIdx.x == 0) {
    ctrl->worst_start = 0;
    ctrl->nv = total;
    ctrl->need = total;
  }
}

// Position of a candidate among nv candidates ordered by (key, candidate index): the number of
// candidates whose (key, index) pair is smaller.  The block's 256 candidates each hold their own pair
// in a register; the pairs of all candidates stream through LDS in tiles of kRankTile, loaded
// cooperatively by `load_pair(q)`, and every thread compares its pair with the whole tile (LDS
// broadcast reads, one 64-bit compare per partner).
constexpr int kRankTile = 1024;

template <class LoadPair>
__device__ inline int rank_by_counting(uint64_t mine, int nv, LoadPair load_pair, uint64_t* tile_lds) {
  int smaller = 0;
  for (int t0 = 0; t0 < nv; t0 += kRankTile) {
    __syncthreads();
    for (int e = threadIdx.x; e < kRankTile; e += blockDim.x) tile_lds[e] = t0 + e < nv ? load_pair(t0 + e) : ~0ull;
    __syncthreads();
    // 16 partners per step, their LDS reads issued together (entries past nv hold all-ones)
    const int lim = min(kRankTile, (int)round_up(nv - t0, 16));
    for (int e = 0; e < lim; e += 16) {
      ulonglong2 v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = *reinterpret_cast<const ulonglong2*>(tile_lds + e + 2 * u);
#pragma unroll
      for (int u = 0; u < 8; ++u) smaller += (v[u].x < mine) + (v[u].y < mine);
    }
  }
  return smaller;
}

// Crowding distance of candidate q from the per-objective sorted positions: the sum over objectives of
// (next - previous) / (last - first) in sorted order, +inf for a candidate that is first or last in any
// objective (non_dominate.py:223-229).  Objectives are added in column order starting from the first
// term, which is what torch's row sum does for the small M of this workload.
__device__ inline float crowding_distance_of(int q, int nv, int m, const int* __restrict__ pos,
                                             const float* __restrict__ sorted_cost, int kstride) {
  bool boundary = false;
  float acc = 0.0f;
  for (int k = 0; k < m; ++k) {
    const float* __restrict__ sc = sorted_cost + (int64_t)k * kstride;
    const int p = pos[(int64_t)k * kstride + q];
    if (p == 0 || p == nv - 1) {
      boundary = true;
    } else {
      const float span = sc[nv - 1] - sc[0];
      const float term = (sc[p + 1] - sc[p - 1]) / span;
      acc = k == 0 ? term : acc + term;
    }
  }
  return boundary ? INFINITY : acc;
}

// out[p, :] = src[order[p], :] for the decision vectors (raw bytes, any dtype), the fitness, the rank
// and the distance.  Rows from n_first on are read from the second part (x2, f2) of a two-part population.
// Rows are copied in 16-, 4- or 1-byte units, a row by 4 to 64 lanes of a wave.
struct GatherArgs {
  const int* order;  // selected rows from position `listed_until` on ...
  const int* listed;  // ... and before it (the rows of the better fronts as the peel listed them) when listed_until > 0
  int topk;
  const uint8_t* x;
  int64_t x_row_stride, x_row_bytes;
  uint8_t* out_x;
  int unit;
  const float* f;
  int64_t f_stride_row, f_stride_col;
  int n_first;
  const uint8_t* x2;
  int64_t x2_row_stride;
  const float* f2;
  int64_t f2_stride_row, f2_stride_col;
  int m;
  float* out_f;
  const int* rank;
  int* out_rank;
  const float* dist;
  float* out_dist;
  int* out_order;
  const Ctrl* ctrl;
  int order_from_peel;  // the host launched nothing that orders the last front: the peel kernel must have (Ctrl.tail_done)
  int* outcome;  // pinned host memory or null: 1 when the peel kernel has ordered the last front of this call, else 2
  // pinned host memory or null: whether front 0 (front0_size rows) held the front0_enough rows that this call keeps --
  // 2: no, 1: yes, 3: yes, and at the call that wrote the word before as well
  int* front0_note;
  const int* front0_size;
  int front0_enough;
  // several populations in one launch (blockIdx.z): from one population to the next, bytes between the library's
  // buffers and between the decision vectors, elements between the fitness; the outputs are topk rows apart
  int64_t ws_step, x_step, x2_step, f_step, f2_step;
};

__device__ __forceinline__ void to_population(GatherArgs& g) {
  to_population(g.ws_step, g.order, g.listed, g.rank, g.dist, g.ctrl);
  const int64_t b = (int64_t)blockIdx.z;
  if (g.x != nullptr) g.x += b * g.x_step;
  if (g.x2 != nullptr) g.x2 += b * g.x2_step;
  if (g.out_x != nullptr) g.out_x += b * g.topk * g.x_row_bytes;
  g.f += b * g.f_step;
  g.f2 += b * g.f2_step;
  g.out_f += b * g.topk * g.m;
  g.out_rank += b * g.topk;
  g.out_dist += b * g.topk;
  if (g.out_order != nullptr) g.out_order += b * g.topk;
}

// Called by every thread of `blocks` blocks of 256 threads (`block` = the caller's index among them).
// listed_until: positions below it take their row from a.listed instead of a.order.
__device__ inline void gather_body(const GatherArgs& a, int block, int blocks, int listed_until) {
  const int topk = a.topk, m = a.m, unit = a.unit, n_first = a.n_first;
  const uint8_t* __restrict__ x = a.x;
  const uint8_t* __restrict__ x2 = a.x2;
  uint8_t* __restrict__ out_x = a.out_x;
  const int64_t x_row_bytes = a.x_row_bytes;
  float* __restrict__ out_f = a.out_f;
  int* __restrict__ out_rank = a.out_rank;
  float* __restrict__ out_dist = a.out_dist;
  int* __restrict__ out_order = a.out_order;
  if (a.ctrl->err != 0 || (a.order_from_peel != 0 && a.ctrl->tail_done == 0)) {
    // a device-side wait ran out and `order` was not produced: no partial result leaves the call -- rank -1,
    // distance and fitness NaN, order -1, decision vectors all-ones bytes (NaN as floats)
    const int64_t threads = (int64_t)blocks * blockDim.x, t0 = (int64_t)block * blockDim.x + threadIdx.x;
    for (int64_t p = t0; p < topk; p += threads) {
      out_rank[p] = -1;
      out_dist[p] = __uint_as_float(0x7FC00000u);
      if (out_order) out_order[p] = -1;
    }
    for (int64_t e = t0; e < (int64_t)topk * m; e += threads) out_f[e] = __uint_as_float(0x7FC00000u);
    if (x)
      for (int64_t b = t0; b < (int64_t)topk * x_row_bytes; b += threads) out_x[b] = 0xFF;
    return;
  }
  // (for the host's choice of launches at its next call; it reads the word without waiting for anything)
  if (a.outcome != nullptr && block == 0 && threadIdx.x == 0)
    __hip_atomic_store(a.outcome, a.ctrl->tail_done != 0 ? 1 : 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
  if (a.front0_note != nullptr && block == 0 && threadIdx.x == 0) {
    const int before = __hip_atomic_load(a.front0_note, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    const int now = *a.front0_size >= a.front0_enough ? (before == 1 || before == 3 ? 3 : 1) : 2;
    __hip_atomic_store(a.front0_note, now, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
  }
  // A row is copied by g lanes, g = the smallest power of two (4 .. 64) that holds the row's units and its m
  // fitness values: short rows share a wave (a row of 400 bytes in 16-byte units took 25 of 64 lanes).
  const int64_t units = (x ? x_row_bytes : 0) / unit;
  int g = 64;
  while (g > 4 && (g >> 1) >= units && (g >> 1) >= m) g >>= 1;
  const int per_wave = 64 / g;
  const int lane = (threadIdx.x & 63) % g, sub = (threadIdx.x & 63) / g;
  const int64_t waves = (int64_t)blocks * (blockDim.x >> 6);
  for (int64_t p = ((int64_t)block * (blockDim.x >> 6) + (threadIdx.x >> 6)) * per_wave + sub; p < topk;
       p += waves * per_wave) {
    const int64_t src = p < listed_until ? a.listed[p] : a.order[p];
    if (src < 0) {  // an order that a failed sort has poisoned: no row is read through it, the outputs say so
      if (x)
        for (int64_t b = lane; b < x_row_bytes; b += g) out_x[p * x_row_bytes + b] = 0xFF;
      for (int k = lane; k < m; k += g) out_f[p * m + k] = __uint_as_float(0x7FC00000u);
      if (lane == 0) {
        out_rank[p] = -1;
        out_dist[p] = __uint_as_float(0x7FC00000u);
        if (out_order) out_order[p] = -1;
      }
      continue;
    }
    const bool second = src >= n_first;  // rows of the second part of a two-part population
    if (x) {
      const uint8_t* __restrict__ s = second ? x2 + (src - n_first) * a.x2_row_stride : x + src * a.x_row_stride;
      uint8_t* __restrict__ d = out_x + p * x_row_bytes;
      if (unit == 16) {
        for (int64_t b = lane * 16; b < x_row_bytes; b += g * 16)
          *reinterpret_cast<uint4*>(d + b) = *reinterpret_cast<const uint4*>(s + b);
      } else if (unit == 4) {
        for (int64_t b = lane * 4; b < x_row_bytes; b += g * 4)
          *reinterpret_cast<uint32_t*>(d + b) = *reinterpret_cast<const uint32_t*>(s + b);
      } else {
        for (int64_t b = lane; b < x_row_bytes; b += g) d[b] = s[b];
      }
    }
    for (int k = lane; k < m; k += g)
      out_f[p * m + k] = second ? a.f2[(src - n_first) * a.f2_stride_row + k * a.f2_stride_col]
                                : a.f[src * a.f_stride_row + k * a.f_stride_col];
    if (lane == 0) {
      out_rank[p] = a.rank[src];
      out_dist[p] = a.dist[src];
      if (out_order) out_order[p] = (int)src;
    }
  }
}

// Winner of every tournament: the candidate that comes first when the tournament's candidates are
// ordered by the LAST key, ties by the key before it, ..., ties by position in the tournament, with NaN
// after every number and signed zeros tied (src/evox/operators/selection/tournament_selection.py:8-29:
// lexsort over the unbound key columns, then column 0).  One thread per tournament.
// fit is (candidates, nkeys) with strides in elements; parents is (n_round, tsize) int64, contiguous.
__global__ __launch_bounds__(256) void tournament_pick_kernel(const int64_t* __restrict__ parents, int64_t n_round, int tsize,
                                                              const float* __restrict__ fit, int64_t stride_row,
                                                              int64_t stride_col, int nkeys, int64_t* __restrict__ out) {
  for (int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; r < n_round; r += (int64_t)gridDim.x * blockDim.x) {
    const int64_t* __restrict__ row = parents + r * tsize;
    int64_t best = row[0];
    for (int t = 1; t < tsize; ++t) {
      const int64_t cand = row[t];
      // strictly better than the current best? (equal on every key keeps the earlier position)
      bool better = false;
      for (int k = nkeys - 1; k >= 0; --k) {
        const uint32_t a = ordered_key(fit[cand * stride_row + k * stride_col]);
        const uint32_t b = ordered_key(fit[best * stride_row + k * stride_col]);
        if (a != b) {
          better = a < b;
          break;
        }
      }
      if (better) best = cand;
    }
    out[r] = best;
  }
}

// The same tournaments on keys that lie in up to four arrays of their own -- what the caller of the reference passes
// (a list of tensors, which the reference stacks: tournament_selection.py:23) -- so that no stacked copy is made.
// kind 0: float32; kind 1: int32, compared as the float32 it converts to (the stack's type promotion).
struct TournamentKeys {
  const void* key[4];
  int64_t stride[4];
  int kind[4];
  int nkeys;
};

__device__ inline uint32_t tournament_key_of(const void* base, int kind, int64_t at) {
  return ordered_key(kind == 0 ? static_cast<const float*>(base)[at] : (float)static_cast<const int*>(base)[at]);
}

__global__ __launch_bounds__(256) void tournament_pick_keys_kernel(const int64_t* __restrict__ parents, int64_t n_round, int tsize,
                                                                   TournamentKeys keys, int64_t* __restrict__ out) {
  for (int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; r < n_round; r += (int64_t)gridDim.x * blockDim.x) {
    const int64_t* __restrict__ row = parents + r * tsize;
    int64_t best = row[0];
    for (int t = 1; t < tsize; ++t) {
      const int64_t cand = row[t];
      bool better = false, decided = false;
#pragma unroll
      for (int k = 3; k >= 0; --k) {  // (constant indices into the argument struct)
        if (k >= keys.nkeys || decided) continue;
        const uint32_t a = tournament_key_of(keys.key[k], keys.kind[k], cand * keys.stride[k]);
        const uint32_t b = tournament_key_of(keys.key[k], keys.kind[k], best * keys.stride[k]);
        if (a != b) {
          better = a < b;
          decided = true;
        }
      }
      if (better) best = cand;
    }
    out[r] = best;
  }
}

}  // namespace evx
