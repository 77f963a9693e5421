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
                                                                   unsigned spin_limit) {
  extern __shared__ uint64_t finish_lds[];
  __shared__ int base[256];
  __shared__ int scratch[kRadixThreads];
  if (coherent_load(&ctrl->err) != 0) return;
  const int nv = ctrl->nv;
  const int* __restrict__ list = list_base + ctrl->worst_start;
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
    if (threadIdx.x == 0) ctrl->radix_epoch += 1;  // nobody reads it again in this kernel
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
                                                                     unsigned spin_limit, int want_order) {
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
      if (threadIdx.x == 0) ctrl->radix_epoch += 1;
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
