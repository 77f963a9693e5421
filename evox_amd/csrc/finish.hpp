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

// A barrier of all `target` workgroups of a resident grid on the counter Ctrl.reserved[which] (zero at the start of the
// call; used once).  False when the bounded wait ran out (Ctrl.err is set then).
// The code on either side exchanges its results (positions, sorted costs, distances, the order) through plain stores
// and loads, which are coherent between kernels but not between the dies of one kernel: the die's L2 is written back
// before the workgroup arrives and its caches are dropped after it leaves.  A write-back or an invalidation works on
// the whole cache, whichever wave asks for it, and costs the same every time (1024 threads of 256 workgroups each
// asking: 65 us per barrier), so one wave of the workgroup asks, once every wave's own stores have arrived in the L2.
__device__ inline bool counter_barrier(Ctrl* ctrl, int which, int target, unsigned spin_limit, int* scratch) {
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  if (threadIdx.x == 0) {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
    __hip_atomic_fetch_add(&ctrl->reserved[which], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const bool seen = bounded_wait([&] { return coherent_load(&ctrl->reserved[which]) >= target; }, spin_limit);
    if (!seen) coherent_store(&ctrl->err, kErrBarrierTimeout);
    scratch[0] = seen;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
  }
  __syncthreads();
  const bool fine = scratch[0] != 0;
  __syncthreads();  // scratch is reused
  return fine;
}

// ---- A small last front in one launch.  With a few hundred candidates the two kernels below cost two launches and
// three chains of dependent loads (positions, sorted costs, distance keys) for a few microseconds of work.  Here the
// candidates' (key, candidate) composites and costs of every objective sit in LDS of every workgroup, a candidate is
// taken by sixteen lanes that scan all candidates once per objective for its two neighbours in the objective's order
// (the largest composite below its own, the smallest above: no positions, no sorted array), and the order of the
// distances follows after one grid-wide counter barrier.  Same results as the two kernels: the neighbours of a
// candidate in the stable order by (cost, row index), the span between the first and the last cost, terms added in
// column order.
constexpr int kFusedFrontRows = 2048;
constexpr int kFusedFrontValues = 4096;  // candidates x objectives held in LDS: 12 bytes each
constexpr int kFusedFrontObjectives = 64;
constexpr int kFusedSoloRows = 128;       // up to here one workgroup does it all (450 rows of two objectives in one workgroup: 100 us, in 29: 20)
constexpr size_t kFusedFrontLdsBytes =
    12 * (size_t)kFusedFrontValues + 4 * (size_t)kFusedFrontRows + 16 * kFusedFrontObjectives + 4 * (size_t)kFusedSoloRows;

__device__ inline bool fused_front_applies(int nv, int m) {
  return nv <= kFusedFrontRows && (int64_t)nv * m <= kFusedFrontValues && m <= kFusedFrontObjectives;
}

// mode 1: distances only; mode 2: distances and the selection order.  Called by every thread of every block;
// blockDim.x == kRadixThreads.  lds: kFusedFrontLdsBytes.
__device__ inline void crowd_small_front(const float* __restrict__ xs, int npad, const int* __restrict__ list_base,
                                         Ctrl* __restrict__ ctrl, int m, float* __restrict__ dist, uint32_t* __restrict__ dkey,
                                         int* __restrict__ order, unsigned spin_limit, int mode, uint64_t* lds, int* scratch) {
  const int nv = ctrl->nv, start = ctrl->worst_start, need = ctrl->need;
  const int* __restrict__ list = list_base + start;
  const int tid = threadIdx.x, sub = tid & 15;
  unsigned long long* comp = reinterpret_cast<unsigned long long*>(lds);  // [m][nv]
  float* cost = reinterpret_cast<float*>(comp + kFusedFrontValues);  // [m][nv]
  int* lst = reinterpret_cast<int*>(cost + kFusedFrontValues);       // [nv]
  unsigned long long* ends = reinterpret_cast<unsigned long long*>(lst + kFusedFrontRows);  // [m][2]: first, last composite
  // A front of a few hundred rows is the work of one workgroup: the others would only repeat its loads and then
  // make it wait for them at the barrier below.
  const bool solo = nv <= kFusedSoloRows;
  // ... and a front of up to kFusedFrontRows rows that of as many workgroups as have sixteen candidates each: the
  // barrier below costs every workgroup that arrives a write-back and an invalidation of its die's cache (the 512
  // workgroups of the grid of a population of 200 000 rows: 100 us for a front of 600 rows)
  const int active = solo ? 1 : min((int)gridDim.x, (nv + (int)(blockDim.x >> 4) - 1) / (int)(blockDim.x >> 4));
  if (mode == 2)  // the better fronts keep the order in which they are listed
    for (int i = blockIdx.x * blockDim.x + tid; i < start; i += gridDim.x * blockDim.x) order[i] = list_base[i];
  if ((int)blockIdx.x >= active) return;
  for (int e = tid; e < nv; e += blockDim.x) lst[e] = list[e];
  __syncthreads();
  for (int i = tid; i < nv * m; i += blockDim.x) {
    const int k = i / nv, e = i - k * nv;
    const float c = xs[(int64_t)k * npad + lst[e]];
    cost[i] = c;
    comp[i] = ((unsigned long long)ordered_key(c) << 32) | (unsigned)e;
  }
  __syncthreads();
  // first and last composite of every objective: a wave per objective
  for (int k = tid >> 6; k < m; k += blockDim.x >> 6) {
    unsigned long long lo = ~0ull, hi = 0ull;
    for (int e = tid & 63; e < nv; e += 64) {
      const unsigned long long c = comp[k * nv + e];
      lo = c < lo ? c : lo;
      hi = c > hi ? c : hi;
    }
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const unsigned long long a = ((unsigned long long)__shfl_xor((unsigned)(lo >> 32), off) << 32) | __shfl_xor((unsigned)lo, off);
      const unsigned long long b = ((unsigned long long)__shfl_xor((unsigned)(hi >> 32), off) << 32) | __shfl_xor((unsigned)hi, off);
      lo = a < lo ? a : lo;
      hi = b > hi ? b : hi;
    }
    if ((tid & 63) == 0) {
      ends[2 * k] = lo;
      ends[2 * k + 1] = hi;
    }
  }
  __syncthreads();
  const int groups = active * (blockDim.x >> 4);
  uint32_t* dkey_lds = reinterpret_cast<uint32_t*>(ends + 2 * kFusedFrontObjectives);  // [kFusedSoloRows], solo only
  for (int q = blockIdx.x * (blockDim.x >> 4) + (tid >> 4); q < nv; q += groups) {
    bool boundary = false;
    float acc = 0.0f;
    for (int k = 0; k < m; ++k) {
      const unsigned long long* row = comp + k * nv;
      const unsigned long long mine = row[q];
      unsigned long long below = 0ull, above = ~0ull;  // no composite is zero or all ones
      for (int e0 = sub; e0 < nv; e0 += 8 * 16) {  // eight partners per step, their LDS reads in flight together
        unsigned long long c[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) c[u] = e0 + 16 * u < nv ? row[e0 + 16 * u] : mine;
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          if (c[u] < mine) below = c[u] > below ? c[u] : below;
          if (c[u] > mine) above = c[u] < above ? c[u] : above;
        }
      }
      below = group16_max(below);
      above = group16_min(above);
      if (below == 0ull || above == ~0ull) {
        boundary = true;  // first or last of this objective (non_dominate.py:226-227)
      } else {
        const float* ck = cost + k * nv;
        const float span = ck[(int)(unsigned)ends[2 * k + 1]] - ck[(int)(unsigned)ends[2 * k]];
        const float term = (ck[(int)(unsigned)above] - ck[(int)(unsigned)below]) / span;
        acc = k == 0 ? term : acc + term;
      }
    }
    if (sub == 0) {
      const float d = boundary ? INFINITY : acc;
      dist[lst[q]] = d;
      if (mode == 2) {
        if (solo)
          dkey_lds[q] = ordered_key(-d);
        else
          dkey[q] = ordered_key(-d);
      }
    }
  }
  if (mode != 2) return;
  __syncthreads();
  if (solo) {
    for (int e = tid; e < nv; e += blockDim.x) comp[e] = ((unsigned long long)dkey_lds[e] << 32) | (unsigned)e;
    __syncthreads();
  } else {
    // every block has stored its distance keys
    if (!counter_barrier(ctrl, 0, active, spin_limit, scratch)) return;
    for (int e = tid; e < nv; e += blockDim.x) comp[e] = ((unsigned long long)dkey[e] << 32) | (unsigned)e;
    __syncthreads();
  }
  for (int q = blockIdx.x * (blockDim.x >> 4) + (tid >> 4); q < nv; q += groups) {
    const unsigned long long mine = comp[q];
    int smaller = 0;
    for (int e0 = sub; e0 < nv; e0 += 8 * 16) {
      unsigned long long c[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) c[u] = e0 + 16 * u < nv ? comp[e0 + 16 * u] : ~0ull;
#pragma unroll
      for (int u = 0; u < 8; ++u) smaller += c[u] < mine;
    }
#pragma unroll
    for (int off = 1; off < 16; off <<= 1) smaller += __shfl_xor(smaller, off);
    if (sub == 0 && smaller < need) order[start + smaller] = lst[q];
  }
}

// Per-objective sorted position of every candidate of the last front: pos[k][q], sorted_cost[k][pos].
// Grid: the radix grid (master, idle block, workers; all resident) when the population can have a
// front above kRadixMinCandidates rows, any grid otherwise.  Dynamic LDS: max(kRankTile * 8,
// kRadixLdsBytes) bytes.
struct CrowdArgs {
  const float* xs;  // fitness, structure of arrays in original row order, columns npad apart
  int npad;
  const int* list_base;  // the rows ordered by (rank, row index) as far as peeled
  Ctrl* ctrl;
  int m, kstride;
  int* pos;
  float* sorted_cost;
  RadixBuffers buf;
  unsigned spin_limit;
  SortParam* param;
  int use_orders, fused;
  // The LDS sorter (mid_argsort_slice) for fronts of kMidSortMinCandidates + 1 to kMidArgsortRows rows: 0 = not used;
  // 1 = this launch has it beside everything else (kMidArgsortThreads threads, populations up to kMidArgsortRows);
  // larger populations get two launches: 2 = this one (kMidArgsortThreads threads) orders such a front and nothing
  // else, 3 = this one (kRadixThreads threads) leaves such a front to the other.
  int mid_sort;
  float* dist;
  uint32_t* dkey;
  int* order;
  int64_t ws_step;  // several populations in one launch: bytes from one population's buffers to the next one's
};

__device__ __forceinline__ void to_population(CrowdArgs& a) {
  to_population(a.ws_step, a.xs, a.list_base, a.ctrl, a.pos, a.sorted_cost, a.buf.pairs[0], a.buf.pairs[1], a.buf.table, a.buf.totals,
                a.param, a.dist, a.dkey, a.order);
}

// Whether a last front of nv rows is ordered by workgroups that sort in LDS (the same answer in every workgroup).
// Smaller fronts are ranked by counting, which is quadratic: 2000 candidates x 3 objectives took 67 us that way, on
// the 24 workgroups that the counting keeps busy.
constexpr int kMidSortMinCandidates = 1024;
__device__ inline bool crowd_mid_applies(const CrowdArgs& a, int nv) {
  return (a.mid_sort == 1 || a.mid_sort == 2) && nv > kMidSortMinCandidates && nv <= kMidArgsortRows &&
         blockDim.x == kMidArgsortThreads;
}
// Where the work is split over two launches (mid_sort 2 and 3): whether the one with the LDS sorter orders the front
// by objective (`by_objective`) or by distance.  A front that crowd_small_front takes, or whose per-objective orders
// are read off those of the population, is not the LDS sorter's.
__device__ inline bool crowd_mid_takes(const CrowdArgs& a, int nv, bool by_objective) {
  if (nv <= kMidSortMinCandidates || nv > kMidArgsortRows) return false;
  if (a.fused != 0 && fused_front_applies(nv, a.m)) return false;
  if (by_objective && nv > kRadixMinCandidates && a.use_orders != 0 && a.param->orders_valid != 0) return false;
  return true;
}

// `epochs`: how many epochs of radix barrier generations the control block's counter moves on when the radix path
// has run (1 when the kernel ends after this body; the merged tail kernel passes 0 and moves the counter itself).
// TABLES: 0 = the launch has no LDS sorter (kRadixThreads threads), 1 = its large tables, 2 = its small ones (the host
// goes by the size of the population).
template <int TABLES>
__device__ inline void crowd_sort_body(const CrowdArgs& a, unsigned gen0, int epochs, uint64_t* finish_lds, int* base, int* scratch) {
  const float* __restrict__ xs = a.xs;
  const int npad = a.npad, m = a.m, kstride = a.kstride, use_orders = a.use_orders, fused = a.fused;
  const int* __restrict__ list_base = a.list_base;
  Ctrl* __restrict__ ctrl = a.ctrl;
  int* __restrict__ pos = a.pos;
  float* __restrict__ sorted_cost = a.sorted_cost;
  const RadixBuffers buf = a.buf;
  const unsigned spin_limit = a.spin_limit;
  SortParam* __restrict__ param = a.param;
  float* __restrict__ dist = a.dist;
  uint32_t* __restrict__ dkey = a.dkey;
  int* __restrict__ order = a.order;
  if (coherent_load(&ctrl->err) != 0) return;
  const int nv = ctrl->nv;
  if (a.mid_sort >= 2 && (a.mid_sort == 2) != crowd_mid_takes(a, nv, true)) return;  // the other launch's front
  if (fused != 0 && fused_front_applies(nv, m)) {  // a small front: distances (and order) right here
    crowd_small_front(xs, npad, list_base, ctrl, m, dist, dkey, order, spin_limit, fused, finish_lds, scratch);
    return;
  }
  const int* __restrict__ list = list_base + ctrl->worst_start;
  // a large front of a population whose per-objective orders are at hand is ordered by front_order_*_kernel
  if (nv > kRadixMinCandidates && use_orders && param->orders_valid != 0) return;
  if (nv <= kRadixMinCandidates && !(TABLES != 0 && crowd_mid_applies(a, nv))) {
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
  if (TABLES != 0 && crowd_mid_applies(a, nv)) {
    // a workgroup produces a run of positions of one objective's order from the front's keys in its LDS; nobody waits
    const int nb = (int)gridDim.x;
    const int per_objective = nb >= m ? nb / m : 1;  // workgroups that share an objective
    const int run = ((nv + per_objective - 1) / per_objective + 15) & ~15;
    for (int item = blockIdx.x; item < per_objective * m; item += nb) {
      const int k = item % m, s0 = (item / m) * run;
      if (s0 >= nv) continue;
      const float* __restrict__ col = xs + (int64_t)k * npad;
      mid_argsort_slice<TABLES == 1>(
          finish_lds, nv, s0, s0 + run, [&](int e) { return ordered_key(col[list[e]]); },
          [&](int p, int e) {
            pos[(int64_t)k * kstride + e] = p;
            sorted_cost[(int64_t)k * kstride + p] = col[list[e]];
          });
    }
    return;
  }
  // radix sort, one segment per objective (the host gave this launch the radix grid)
  if (blockIdx.x == 0) {
    radix_master(ctrl, gen0, 12, spin_limit, scratch);
    if (threadIdx.x == 0) {
      ctrl->radix_epoch += epochs;  // nobody reads it again in this kernel
      param->orders_valid = 0;  // the sort has taken the buffer that held them (read at the start of this body only)
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

// after_peel_tail: the peel kernel may have ordered the last front already (Ctrl.tail_done).
// T threads: kRadixThreads, or kMidArgsortThreads where CrowdArgs.mid_sort is set (the radix sort, which is written for
// kRadixThreads, does not run then).
template <int T, int TABLES, bool MANY = false>
__global__ __launch_bounds__(T) void crowd_sort_kernel(CrowdArgs a, int after_peel_tail) {
  extern __shared__ __attribute__((aligned(16))) uint64_t finish_lds[];
  __shared__ int base[256];
  __shared__ int scratch[kRadixThreads];
  if constexpr (MANY) to_population(a);  // several populations in the launch, one per blockIdx.z
  if (after_peel_tail != 0 && a.ctrl->tail_done != 0) return;
  crowd_sort_body<TABLES>(a, radix_generation_base(a.ctrl), 1, finish_lds, base, scratch);
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
template <int TABLES>
__device__ inline void crowd_finish_body(const CrowdArgs& a, int want_order, unsigned gen0, int epochs, uint64_t* finish_lds,
                                         int* base, int* scratch) {
  const int m = a.m, kstride = a.kstride, fused = a.fused;
  const int* __restrict__ list_base = a.list_base;
  Ctrl* __restrict__ ctrl = a.ctrl;
  const int* __restrict__ pos = a.pos;
  const float* __restrict__ sorted_cost = a.sorted_cost;
  const RadixBuffers buf = a.buf;
  const unsigned spin_limit = a.spin_limit;
  SortParam* __restrict__ param = a.param;
  float* __restrict__ dist = a.dist;
  uint32_t* __restrict__ dkey = a.dkey;
  int* __restrict__ order = a.order;
  if (coherent_load(&ctrl->err) != 0) return;
  const int nv = ctrl->nv;
  if (a.mid_sort >= 2 && (a.mid_sort == 2) != crowd_mid_takes(a, nv, false)) return;  // the other launch's front
  if (fused != 0 && fused_front_applies(nv, m)) return;  // crowd_sort_kernel has done it all
  const int start = ctrl->worst_start;
  const int need = ctrl->need;
  const int* __restrict__ list = list_base + start;
  if (nv <= kRadixMinCandidates && !(TABLES != 0 && crowd_mid_applies(a, nv))) {
    // every block derives the distance keys of all candidates in LDS (a few thousand table look-ups);
    // block 0 also stores the distances
    uint32_t* dkey_lds = reinterpret_cast<uint32_t*>(finish_lds);
    uint64_t* tile_lds = finish_lds + kRadixMinCandidates / 2;
    if (!want_order && blockIdx.x != 0) return;
    if (blockIdx.x != 0 && (int64_t)blockIdx.x * blockDim.x >= nv) {
      // no candidate of its own to place: this block only helps to copy the listing of the better fronts (the
      // distance keys below are derived by every block that uses them: a larger grid must not multiply that)
      for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < start; i += gridDim.x * blockDim.x) order[i] = list_base[i];
      return;
    }
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
  if (TABLES != 0 && crowd_mid_applies(a, nv)) {
    // distances by stripes; then, for the order, every workgroup takes all distance keys into its LDS and produces a
    // run of the first `need` positions
    EVX_TRACE(50, 0);
    for (int q = blockIdx.x * blockDim.x + threadIdx.x; q < nv; q += gridDim.x * blockDim.x) {
      const float d = crowding_distance_of(q, nv, m, pos, sorted_cost, kstride);
      dist[list[q]] = d;
      dkey[q] = ordered_key(-d);
    }
    if (!want_order) return;
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < start; i += gridDim.x * blockDim.x) order[i] = list_base[i];
    EVX_TRACE(50, 1);
    if (!counter_barrier(ctrl, 3, (int)gridDim.x, spin_limit, scratch)) return;
    EVX_TRACE(50, 2);
    const int run = ((need + (int)gridDim.x - 1) / (int)gridDim.x + 15) & ~15;
    const int s0 = (int)blockIdx.x * run;
    if (s0 < need)
      mid_argsort_slice<TABLES == 1, 52>(
          finish_lds, nv, s0, min(need, s0 + run),
          // (the key of an infinite distance lies far below those of the finite ones, which would leave them a twentieth
          // of the sorter's buckets: any key below that of -m will do for it, a distance being at most m)
          [&](int e) {
            const uint32_t k = dkey[e];
            return k == 0x007FFFFFu /* ordered_key(-inf) */ ? 0x37FFFFFFu /* ordered_key(-131072) */ : k;
          },
          [&](int p, int e) { order[start + p] = list[e]; });
    EVX_TRACE(50, 3);
    return;
  }
  // large front: distances by stripes, then (for the order) a grid barrier and the radix sort of their keys
  if (blockIdx.x == 0) {
    if (want_order) {
      radix_master(ctrl, gen0, 13, spin_limit, scratch);
      if (threadIdx.x == 0) {
        ctrl->radix_epoch += epochs;
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

template <int T, int TABLES, bool MANY = false>
__global__ __launch_bounds__(T) void crowd_finish_kernel(CrowdArgs a, int want_order, int after_peel_tail) {
  extern __shared__ __attribute__((aligned(16))) uint64_t finish_lds[];
  __shared__ int base[256];
  __shared__ int scratch[kRadixThreads];
  if constexpr (MANY) to_population(a);
  if (after_peel_tail != 0 && a.ctrl->tail_done != 0) return;
  crowd_finish_body<TABLES>(a, want_order, radix_generation_base(a.ctrl), 1, finish_lds, base, scratch);
}

// ---- The ordering of the last front in one launch (crowd_gather_kernel below), for populations whose peel kernel
// orders a small last front itself (Ctrl.tail_done says whether it has: then nothing is left to order).  A launch
// that finds nothing to do still costs as much as a small kernel (about 4.7 us on this device), so the two stages
// share one launch; they are separated by a counter barrier of all blocks.  Grid: that of crowd_sort_kernel (the
// radix grid: master, idle block, workers), resident at once.
__device__ inline bool tail_barrier(Ctrl* ctrl, int target, unsigned spin_limit, int* scratch) {
  return counter_barrier(ctrl, 1, target, spin_limit, scratch);
}

template <bool MANY>
__global__ __launch_bounds__(256) void gather_kernel(GatherArgs g) {
  if constexpr (MANY) to_population(g);
  gather_body(g, blockIdx.x, gridDim.x, 0);
}

// listed: the rows of the better fronts as the peel listed them; positions below Ctrl.worst_start take their row
// from there when the peel kernel has ordered the last front (it then leaves only that front's part of `order`).
template <bool MANY>
__global__ __launch_bounds__(256) void gather_after_peel_kernel(GatherArgs g) {
  if constexpr (MANY) to_population(g);
  gather_body(g, blockIdx.x, gridDim.x, g.ctrl->err == 0 && g.ctrl->tail_done != 0 ? g.ctrl->worst_start : 0);
}

// Both ordering stages and the gather of the selected rows behind them.  When the peel kernel has ordered the last
// front -- the usual case where this kernel is launched -- the gather is all that is left, and it starts at once: one
// launch after the peel instead of two or three.  Otherwise the order is complete when every block has passed the
// second round of the barrier counter that separates the two ordering stages.  After a failed wait the gather writes
// no rows (it looks at Ctrl.err).
template <int T, int TABLES, bool MANY>
__global__ __launch_bounds__(T) void crowd_gather_kernel(CrowdArgs a, GatherArgs g) {
  extern __shared__ __attribute__((aligned(16))) uint64_t finish_lds[];
  __shared__ int base[256];
  __shared__ int scratch[kRadixThreads];
  if constexpr (MANY) {  // several populations in the launch, one per blockIdx.z
    to_population(a);
    to_population(g);
  }
  Ctrl* ctrl = a.ctrl;
  if (coherent_load(&ctrl->err) != 0) {
    gather_body(g, blockIdx.x, gridDim.x, 0);
    return;
  }
  if (ctrl->tail_done != 0) {
    gather_body(g, blockIdx.x, gridDim.x, ctrl->worst_start);
    return;
  }
  const unsigned gen0 = radix_generation_base(ctrl);
  crowd_sort_body<TABLES>(a, gen0, 0, finish_lds, base, scratch);
  if (tail_barrier(ctrl, (int)gridDim.x, a.spin_limit, scratch))
    crowd_finish_body<TABLES>(a, 1, gen0 + 16u, 0, finish_lds, base, scratch);
  if (blockIdx.x == 0 && threadIdx.x == 0) ctrl->radix_epoch += 2;  // both bodies may have run a radix sort
  counter_barrier(ctrl, 1, 2 * (int)gridDim.x, a.spin_limit, scratch);
  gather_body(g, blockIdx.x, gridDim.x, 0);
}

}  // namespace evx
