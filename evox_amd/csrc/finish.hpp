// The two kernels that follow the peeling: the per-objective ordering of the last front, and its
// crowding distances together with the index-stable top-k.
//
// Reference semantics:
//   crowding_distance            src/evox/operators/selection/non_dominate.py:198-231
//   lexsort (stable, last key primary)   src/evox/utils/jit_fix_operator.py:246-252
//   nd_environmental_selection   non_dominate.py:250-254
//
// The size of the last front is only known on the device, and two orderings exist for it: ranking by
// counting (crowd.hpp: one pass, no dependent steps) for fronts of at most kRadixMinCandidates rows and
// the segmented radix sort (radix.hpp: persistent, grid barriers) above.  Each kernel here holds both
// and picks one when it runs, so that a selection costs two launches after the peeling instead of one
// launch per variant and stage.
#pragma once

#include "crowd.hpp"
#include "order.hpp"
#include "radix.hpp"

namespace evx {

// Per-objective sorted position of every candidate of the last front: pos[k][q], sorted_cost[k][pos].
// Grid: the radix grid (master, idle block, workers; all resident) when the population can have a
// front above kRadixMinCandidates rows, any grid otherwise.  Dynamic LDS: max(kRankTile * 8,
// kRadixLdsBytes) bytes.
__global__ __launch_bounds__(kRadixThreads) void crowd_sort_kernel(const float* __restrict__ xs, int npad,
                                                                   const int* __restrict__ list_base, Ctrl* __restrict__ ctrl,
                                                                   int m, int kstride, int* __restrict__ pos,
                                                                   float* __restrict__ sorted_cost, RadixBuffers buf,
                                                                   unsigned spin_limit, SortParam* __restrict__ param,
                                                                   int use_orders) {
  extern __shared__ uint64_t finish_lds[];
  __shared__ int base[256];
  __shared__ int scratch[kRadixThreads];
  if (coherent_load(&ctrl->err) != 0) return;
  const int nv = ctrl->nv;
  const int* __restrict__ list = list_base + ctrl->worst_start;
  // a large front of a population whose per-objective orders are at hand is ordered by front_order_*_kernel
  if (nv > kRadixMinCandidates && use_orders && param->orders_valid != 0) return;
  if (nv <= kRadixMinCandidates) {
    // ranking by counting: one work item per (256 candidates, objective)
    const int qblocks = (nv + (int)blockDim.x - 1) / (int)blockDim.x;
    for (int item = blockIdx.x; item < qblocks * m; item += gridDim.x) {
      const int k = item / qblocks;
      const int q = (item - k * qblocks) * (int)blockDim.x + (int)threadIdx.x;
      const float* __restrict__ col = xs + (int64_t)k * npad;
      auto pair_of = [&](int e) { return ((uint64_t)ordered_key(col[list[e]]) << 32) | (uint32_t)e; };
      const float cost = q < nv ? col[list[q]] : 0.0f;
      const uint64_t mine = q < nv ? (((uint64_t)ordered_key(cost) << 32) | (uint32_t)q) : 0ull;
      const int p = rank_by_counting(mine, nv, pair_of, finish_lds);
      if (q < nv) {
        pos[(int64_t)k * kstride + q] = p;
        sorted_cost[(int64_t)k * kstride + p] = cost;
      }
    }
    return;
  }
  // radix sort, one segment per objective (the host gave this launch the radix grid)
  const unsigned gen0 = radix_generation_base(ctrl);
  if (blockIdx.x == 0) {
    radix_master(ctrl, gen0, 12, spin_limit, scratch);
    if (threadIdx.x == 0) {
      ctrl->radix_epoch += 1;  // nobody reads it again in this kernel
      param->orders_valid = 0;  // the sort has taken the buffer that held them (read at the start of this kernel only)
    }
    return;
  }
  if (blockIdx.x < kFirstSweeper) return;
  const int workers = gridDim.x - kFirstSweeper;
  const int wb = (int)blockIdx.x - kFirstSweeper;
  auto initial = [&](int k, int q) {
    return ((unsigned long long)ordered_key(xs[(int64_t)k * npad + list[q]]) << 32) | (unsigned)q;
  };
  if (!radix_sort_segments(buf, m, nv, initial, ctrl, gen0, spin_limit, reinterpret_cast<int*>(finish_lds), base, scratch)) return;
  for (int k = 0; k < m; ++k)
    for (int p = wb * blockDim.x + threadIdx.x; p < nv; p += workers * blockDim.x) {
      const unsigned long long pr = coherent_load(&buf.pairs[0][(int64_t)k * buf.kstride + p]);
      const int q = (int)(unsigned)(pr & 0xFFFFFFFFull);
      pos[(int64_t)k * buf.kstride + q] = p;
      sorted_cost[(int64_t)k * buf.kstride + p] = xs[(int64_t)k * npad + list[q]];
    }
}

// ---- The same per-objective order of a large last front, taken from the orders of the whole population that
// objective_order_kernel has left in the radix buffer: the candidates of the front, in the order in which they appear
// among all rows of objective k (value ascending, equal values by original index = by candidate number), are the
// front in its own order; a candidate's position is the number of candidates before it.  Three launches with no
// dependence between workgroups inside a launch; each does nothing unless the front is large and the orders are valid.
constexpr int kFrontOrderSpan = 1024;  // positions per workgroup

__device__ inline bool front_orders_apply(const Ctrl* ctrl, const SortParam* param) {
  return ctrl->err == 0 && param->orders_valid != 0 && ctrl->nv > kRadixMinCandidates;
}

// number[list[q]] = q: the candidate number of every row of the front.
__global__ __launch_bounds__(256) void front_number_kernel(const int* __restrict__ list_base, const Ctrl* __restrict__ ctrl,
                                                           const SortParam* __restrict__ param, int* __restrict__ number) {
  if (!front_orders_apply(ctrl, param)) return;
  const int nv = ctrl->nv;
  const int* __restrict__ list = list_base + ctrl->worst_start;
  for (int q = blockIdx.x * blockDim.x + threadIdx.x; q < nv; q += gridDim.x * blockDim.x) number[list[q]] = q;
}

// per_span[k * gridDim.x + b] = candidates among positions b * kFrontOrderSpan ... of objective k = blockIdx.y.
__global__ __launch_bounds__(256) void front_order_count_kernel(const unsigned long long* __restrict__ sorted, int kstride, int n,
                                                                const int* __restrict__ rank, const Ctrl* __restrict__ ctrl,
                                                                const SortParam* __restrict__ param, int* __restrict__ per_span) {
  __shared__ int total;
  if (!front_orders_apply(ctrl, param)) return;
  const int worst = ctrl->worst;
  const int k = blockIdx.y;
  if (threadIdx.x == 0) total = 0;
  __syncthreads();
  int mine = 0;
#pragma unroll
  for (int u = 0; u < kFrontOrderSpan / 256; ++u) {
    const int p = blockIdx.x * kFrontOrderSpan + u * 256 + (int)threadIdx.x;
    if (p < n) mine += rank[(int)(unsigned)(sorted[(int64_t)k * kstride + p] & 0xFFFFFFFFull)] == worst ? 1 : 0;
  }
  mine = wave_sum(mine);
  if ((threadIdx.x & 63) == 0 && mine != 0) atomicAdd(&total, mine);
  __syncthreads();
  if (threadIdx.x == 0) per_span[k * gridDim.x + blockIdx.x] = total;
}

// pos[k][number] and sorted_cost[k][position] of the candidates among the positions of this workgroup.
__global__ __launch_bounds__(256) void front_order_place_kernel(const unsigned long long* __restrict__ sorted, int kstride, int n,
                                                                const int* __restrict__ rank, const Ctrl* __restrict__ ctrl,
                                                                const SortParam* __restrict__ param,
                                                                const int* __restrict__ per_span, const int* __restrict__ number,
                                                                const float* __restrict__ xs, int npad, int* __restrict__ pos,
                                                                float* __restrict__ sorted_cost) {
  __shared__ int before_span;
  __shared__ int wave_count[kFrontOrderSpan / 256][4];
  if (!front_orders_apply(ctrl, param)) return;
  const int worst = ctrl->worst;
  const int k = blockIdx.y;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  constexpr int U = kFrontOrderSpan / 256;
  // the rows at this thread's positions and whether they are candidates: all loads of a step before any use
  int row[U];
  bool is[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int p = blockIdx.x * kFrontOrderSpan + u * 256 + (int)threadIdx.x;
    row[u] = p < n ? (int)(unsigned)(sorted[(int64_t)k * kstride + p] & 0xFFFFFFFFull) : -1;
  }
#pragma unroll
  for (int u = 0; u < U; ++u) is[u] = row[u] >= 0 && rank[row[u]] == worst;
  if (threadIdx.x == 0) before_span = 0;
  __syncthreads();
  int mine = 0;
  for (int b = threadIdx.x; b < (int)blockIdx.x; b += 256) mine += per_span[k * gridDim.x + b];
  mine = wave_sum(mine);
  if (lane == 0 && mine != 0) atomicAdd(&before_span, mine);
  int in_wave[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const uint64_t members = __builtin_amdgcn_ballot_w64(is[u]);
    in_wave[u] = __popcll(members & ((1ull << lane) - 1ull));
    if (lane == 0) wave_count[u][wave] = __popcll(members);
  }
  __syncthreads();
  int number_of[U];
  float cost[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    number_of[u] = is[u] ? number[row[u]] : 0;
    cost[u] = is[u] ? xs[(int64_t)k * npad + row[u]] : 0.0f;
  }
  int running = before_span;  // candidates before the 256 positions of step u
#pragma unroll
  for (int u = 0; u < U; ++u) {
    int place = running + in_wave[u];
    for (int v = 0; v < wave; ++v) place += wave_count[u][v];
    if (is[u]) {
      pos[(int64_t)k * kstride + number_of[u]] = place;
      sorted_cost[(int64_t)k * kstride + place] = cost[u];
    }
    running += wave_count[u][0] + wave_count[u][1] + wave_count[u][2] + wave_count[u][3];
  }
}

// Crowding distance of every candidate of the last front (written by original index) and, when
// `want_order` is set, the selection order: the better fronts as listed, then the `need` candidates
// that come first by (distance descending, NaN after every number, row index) -- jit_fix_operator.py:246-252
// applied to non_dominate.py:253.  Same grid rule as crowd_sort_kernel.  Dynamic LDS:
// kRadixMinCandidates * 4 + kRankTile * 8 bytes.
__global__ __launch_bounds__(kRadixThreads) void crowd_finish_kernel(const int* __restrict__ list_base, Ctrl* __restrict__ ctrl,
                                                                     int m, const int* __restrict__ pos,
                                                                     const float* __restrict__ sorted_cost, int kstride,
                                                                     float* __restrict__ dist, uint32_t* __restrict__ dkey,
                                                                     int* __restrict__ order, RadixBuffers buf,
                                                                     unsigned spin_limit, int want_order,
                                                                     SortParam* __restrict__ param) {
  extern __shared__ uint64_t finish_lds[];
  __shared__ int base[256];
  __shared__ int scratch[kRadixThreads];
  if (coherent_load(&ctrl->err) != 0) return;
  const int nv = ctrl->nv;
  const int start = ctrl->worst_start;
  const int need = ctrl->need;
  const int* __restrict__ list = list_base + start;
  if (nv <= kRadixMinCandidates) {
    // every block derives the distance keys of all candidates in LDS (a few thousand table look-ups);
    // block 0 also stores the distances
    uint32_t* dkey_lds = reinterpret_cast<uint32_t*>(finish_lds);
    uint64_t* tile_lds = finish_lds + kRadixMinCandidates / 2;
    if (!want_order && blockIdx.x != 0) return;
    for (int q = threadIdx.x; q < nv; q += blockDim.x) {
      const float d = crowding_distance_of(q, nv, m, pos, sorted_cost, kstride);
      if (blockIdx.x == 0) dist[list[q]] = d;
      dkey_lds[q] = ordered_key(-d);
    }
    __syncthreads();
    if (!want_order) return;
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < start; i += gridDim.x * blockDim.x) order[i] = list_base[i];
    auto pair_of = [&](int e) { return ((uint64_t)dkey_lds[e] << 32) | (uint32_t)e; };
    for (int q0 = blockIdx.x * blockDim.x; q0 < nv; q0 += gridDim.x * blockDim.x) {
      const int q = q0 + threadIdx.x;
      const uint64_t mine = q < nv ? pair_of(q) : 0ull;
      const int p = rank_by_counting(mine, nv, pair_of, tile_lds);
      if (q < nv && p < need) order[start + p] = list[q];
    }
    return;
  }
  // large front: distances by stripes, then (for the order) a grid barrier and the radix sort of their keys
  const unsigned gen0 = radix_generation_base(ctrl);
  if (blockIdx.x == 0) {
    if (want_order) {
      radix_master(ctrl, gen0, 13, spin_limit, scratch);
      if (threadIdx.x == 0) {
        ctrl->radix_epoch += 1;
        param->orders_valid = 0;  // the sort of the distance keys has taken the buffer that held the orders
      }
    }
    return;
  }
  if (blockIdx.x < kFirstSweeper) return;
  const int workers = gridDim.x - kFirstSweeper;
  const int wb = (int)blockIdx.x - kFirstSweeper;
  for (int q = wb * blockDim.x + threadIdx.x; q < nv; q += workers * blockDim.x) {
    const float d = crowding_distance_of(q, nv, m, pos, sorted_cost, kstride);
    dist[list[q]] = d;
    coherent_store(&dkey[q], ordered_key(-d));
  }
  if (!want_order) return;
  int dummy = 0;
  if (!sweeper_barrier(ctrl, gen0 + 1, 0, &dummy, spin_limit, scratch)) return;
  for (int i = wb * blockDim.x + threadIdx.x; i < start; i += workers * blockDim.x) order[i] = list_base[i];
  auto initial = [&](int, int q) { return ((unsigned long long)coherent_load(&dkey[q]) << 32) | (unsigned)q; };
  if (!radix_sort_segments(buf, 1, nv, initial, ctrl, gen0 + 1, spin_limit, reinterpret_cast<int*>(finish_lds), base, scratch)) return;
  for (int p = wb * blockDim.x + threadIdx.x; p < need; p += workers * blockDim.x) {
    const unsigned long long pr = coherent_load(&buf.pairs[0][p]);
    order[start + p] = list[(int)(unsigned)(pr & 0xFFFFFFFFull)];
  }
}

}  // namespace evx
