// Relabelling of the population by ascending row key ("slots").
//
// key(i) = sum_k w_k ordered_key(x[i,k]) (w_k > 0: key_weight in dominance.hpp) is strictly smaller for a dominator than for the row it
// dominates (every term is <=, one is <, and NaN rows dominate nothing), so after sorting the rows by
// (key, original index) every dominance pair has slot(i) < slot(j): the bit matrix built in slot
// space is strictly lower triangular.  That halves the dominance work, bounds every row scan by the
// row's own slot, and makes "the highest unranked dominator" a near-perfect witness for the peel
// (rows of large key lie in deep fronts).  Results never depend on the labelling: ranks are written
// back by original index and fronts are listed in original-index order.
//
// The sort is an exact bucket sort in four small kernels: histogram of a monotone quantisation of the
// key, exclusive scan of the histogram, unordered scatter of the rows into their bucket ranges
// (atomics), and an exact placement inside each bucket by counting the members that precede the row in
// (key, original index) order.  The outcome is deterministic although the scatter is not.
#pragma once

#include "common.hpp"

namespace evx {

struct SortParam {
  unsigned long long kmin;
  int shift;
  int buckets;
  int nonfinite;  // some fitness value of the population is NaN or infinite
  int totals_valid;  // the dominance stage has left popcount and highest word of every row (zero after the slot sort)
  int orders_valid;  // the radix buffer holds every objective's (key, original index) pairs in ascending order (zero after the slot sort)
};

__device__ inline int bucket_of(uint64_t key, const SortParam& p) { return (int)((key - p.kmin) >> p.shift); }

// Reduces the per-block (min key, max key, non-finite flag) partials written by prepare_kernel and derives the
// quantisation: (key - kmin) >> shift < buckets.  Every block of the histogram kernel calls it.
__device__ inline SortParam make_sort_param(const unsigned long long* __restrict__ partials, int nparts, int buckets,
                                            unsigned long long* lds2) {
  if (threadIdx.x < 64) {
    unsigned long long lo = ~0ull, hi = 0ull, bad = 0ull;
    for (int p = threadIdx.x; p < nparts; p += 64) {
      const unsigned long long a = partials[3 * p], b = partials[3 * p + 1];
      lo = a < lo ? a : lo;
      hi = b > hi ? b : hi;
      bad |= partials[3 * p + 2];
    }
    bad = __builtin_amdgcn_ballot_w64(bad != 0ull);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const unsigned long long a = __shfl_xor(lo, off), b = __shfl_xor(hi, off);
      lo = a < lo ? a : lo;
      hi = b > hi ? b : hi;
    }
    if (threadIdx.x == 0) {
      lds2[0] = lo;
      lds2[1] = hi;
      lds2[2] = bad;
    }
  }
  __syncthreads();
  SortParam sp;
  sp.kmin = lds2[0];
  sp.buckets = buckets;
  sp.nonfinite = lds2[2] != 0ull;
  sp.totals_valid = 0;
  sp.orders_valid = 0;
  const unsigned long long span = lds2[1] >= lds2[0] ? lds2[1] - lds2[0] : 0ull;
  int shift = 0;
  while (shift < 63 && (span >> shift) >= (unsigned long long)buckets) ++shift;
  sp.shift = shift;
  return sp;
}

// (MANY, here and below: several populations in the launch, one per blockIdx.z; the instance for one population is
// compiled without the pointer moves)
template <bool MANY>
__global__ __launch_bounds__(256) void bucket_hist_kernel(const uint64_t* __restrict__ key, int n,
                                                          const unsigned long long* __restrict__ partials, int nparts,
                                                          int buckets, int* __restrict__ hist, SortParam* __restrict__ param_out,
                                                          int64_t ws_step) {
  __shared__ unsigned long long lds2[3];
  if constexpr (MANY) to_population(ws_step, key, partials, hist, param_out);
  const SortParam sp = make_sort_param(partials, nparts, buckets, lds2);
  if (blockIdx.x == 0 && threadIdx.x == 0) *param_out = sp;
  const int lane = threadIdx.x & 63;
  for (int i0 = blockIdx.x * blockDim.x; i0 < n; i0 += gridDim.x * blockDim.x) {
    const int i = i0 + threadIdx.x;
    const int b = i < n ? bucket_of(key[i], sp) : -1;
    // Thousands of equal rows (a penalty value for every infeasible row, say) meet in one bucket: the lanes of a wave
    // that share a bucket with one of its first three lanes send one addition between them, so that the additions to
    // a crowded bucket do not queue up one by one (20 000 equal rows: 229 us otherwise).
    uint64_t todo = __builtin_amdgcn_ballot_w64(b >= 0);
    for (int round = 0; round < 3 && todo != 0ull; ++round) {
      const int leader = __builtin_amdgcn_readlane(b, __ffsll((unsigned long long)todo) - 1);
      const uint64_t same = __builtin_amdgcn_ballot_w64(b == leader) & todo;
      if (lane == __ffsll((unsigned long long)same) - 1) atomicAdd(&hist[leader], __popcll(same));
      todo &= ~same;
    }
    if ((todo >> lane) & 1ull) atomicAdd(&hist[b], 1);
  }
}

// start[b] = exclusive prefix of hist, start[buckets] = n; cursor = copy of start.
// One block of 256 threads per 1024 bins (at most 64 blocks, all resident): each block adds up its
// bins, publishes (1 << 32 | total) in its flag, adds the totals of the blocks before it as they appear
// (the flags start at zero), and then scans its own bins.  A block only ever waits for blocks of
// lower index, which are dispatched before it and wait for nobody above them, so the wait ends; it is
// bounded all the same (kScanSpinLimit ticks of 10 ns), and running out sets the error flag, on which every
// later kernel of the call returns without touching the half-built tables.
constexpr unsigned kScanSpinLimit = 1u << 24;

template <bool MANY>
__global__ __launch_bounds__(256) void bucket_scan_kernel(const int* __restrict__ hist, int buckets, int* __restrict__ start,
                                                          int* __restrict__ cursor, unsigned long long* __restrict__ flags,
                                                          Ctrl* __restrict__ ctrl, int64_t ws_step) {
  __shared__ int wave_tot[4];
  if constexpr (MANY) to_population(ws_step, hist, start, cursor, flags, ctrl);
  __shared__ int base_lds;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int b0 = blockIdx.x * 1024 + threadIdx.x * 4;
  const int4 v = *reinterpret_cast<const int4*>(hist + b0);
  const int mine = v.x + v.y + v.z + v.w;
  int incl = mine;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const int up = __shfl_up(incl, off);
    if (lane >= off) incl += up;
  }
  if (lane == 63) wave_tot[wave] = incl;
  __syncthreads();
  const int block_total = wave_tot[0] + wave_tot[1] + wave_tot[2] + wave_tot[3];
  if (threadIdx.x == 0)
    __hip_atomic_store(&flags[blockIdx.x], (1ull << 32) | (unsigned)block_total, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  // the first wave gathers the totals of the preceding blocks (at most 63)
  if (wave == 0) {
    int before = 0;
    if (lane < (int)blockIdx.x) {
      unsigned long long f = 0;
      unsigned spins = 0;
      WaitBound bound(kScanSpinLimit);
      while (((f = __hip_atomic_load(&flags[lane], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) >> 32) == 0) {
        if (bound.expired(++spins)) {
          __hip_atomic_store(&ctrl->err, kErrBarrierTimeout, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          break;
        }
        __builtin_amdgcn_s_sleep(1);
      }
      before = (int)(unsigned)(f & 0xFFFFFFFFull);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) before += __shfl_xor(before, off);
    if (lane == 0) base_lds = before;
  }
  __syncthreads();
  int run = base_lds + incl - mine;
  for (int w = 0; w < wave; ++w) run += wave_tot[w];
  int4 o;
  o.x = run; run += v.x;
  o.y = run; run += v.y;
  o.z = run; run += v.z;
  o.w = run; run += v.w;
  *reinterpret_cast<int4*>(start + b0) = o;
  *reinterpret_cast<int4*>(cursor + b0) = o;
  if (blockIdx.x == gridDim.x - 1 && threadIdx.x == 255) start[buckets] = run;
}

template <bool MANY>
__global__ __launch_bounds__(256) void bucket_scatter_kernel(const uint64_t* __restrict__ key, int n,
                                                             const SortParam* __restrict__ param, int* __restrict__ cursor,
                                                             int* __restrict__ members, uint64_t* __restrict__ member_key,
                                                             const Ctrl* __restrict__ ctrl, int64_t ws_step) {
  if constexpr (MANY) to_population(ws_step, key, param, cursor, members, member_key, ctrl);
  if (ctrl->err != 0) return;
  const SortParam sp = *param;
  const int lane = threadIdx.x & 63;
  for (int i0 = blockIdx.x * blockDim.x; i0 < n; i0 += gridDim.x * blockDim.x) {
    const int i = i0 + threadIdx.x;
    const uint64_t ki = i < n ? key[i] : 0ull;
    const int b = i < n ? bucket_of(ki, sp) : -1;
    // (as in the histogram: the lanes that share a bucket with one of the wave's first three take their places with
    // one addition between them; the groups are found first and all additions go out together, so that the wave waits
    // for one round trip to memory, as it did with one addition per lane)
    uint64_t todo = __builtin_amdgcn_ballot_w64(b >= 0);
    uint64_t group[3] = {0ull, 0ull, 0ull};
    int first[3] = {0, 0, 0};
#pragma unroll
    for (int round = 0; round < 3; ++round) {
      if (todo == 0ull) break;
      const int leader = __builtin_amdgcn_readlane(b, __ffsll((unsigned long long)todo) - 1);
      group[round] = __builtin_amdgcn_ballot_w64(b == leader) & todo;
      first[round] = __ffsll((unsigned long long)group[round]) - 1;
      todo &= ~group[round];
    }
    const uint64_t me = 1ull << lane;
    int count = (todo & me) ? 1 : 0;  // a lane of no group adds for itself
#pragma unroll
    for (int round = 0; round < 3; ++round)
      if (group[round] != 0ull && lane == first[round]) count = __popcll(group[round]);
    int at = 0;
    if (count != 0) at = atomicAdd(&cursor[b], count);
    int p = at;
#pragma unroll
    for (int round = 0; round < 3; ++round) {
      if (group[round] == 0ull) continue;
      const int base = __builtin_amdgcn_readlane(at, first[round]);
      if (group[round] & me) p = base + __popcll(group[round] & (me - 1ull));
    }
    if (i < n) {
      members[p] = i;
      member_key[p] = ki;  // beside the index, so that the placing kernel reads a bucket without a dependent load
    }
  }
}

constexpr int kPlaceLarge = 512;  // a bucket of more members goes through LDS once per workgroup, not through memory once per row
constexpr int kPlaceTile = 1024;  // its members in LDS at a time

// Exact slot of every row: bucket start + number of bucket members that precede it by (key, index).
// Writes the slot-ordered copies of the fitness (structure of arrays, NaN padding up to npad), of
// the keys (all-ones padding), the slot -> original index table (-1 padding) and its inverse.
template <bool MANY>
__global__ __launch_bounds__(256) void bucket_place_kernel(const float* __restrict__ xs, int n,
                                                           int m, int npad, const SortParam* __restrict__ param,
                                                           const int* __restrict__ start, const int* __restrict__ members,
                                                           const uint64_t* __restrict__ member_key,
                                                           uint64_t* __restrict__ key_sorted, uint32_t* __restrict__ kid_sorted,
                                                           float* __restrict__ xs_sorted, int* __restrict__ orig_of,
                                                           int* __restrict__ slot_of, const Ctrl* __restrict__ ctrl, int64_t ws_step) {
  if constexpr (MANY) to_population(ws_step, xs, param, start, members, member_key, key_sorted, kid_sorted, xs_sorted, orig_of, slot_of, ctrl);
  if (ctrl->err != 0) return;
  const SortParam sp = *param;
  __shared__ __attribute__((aligned(16))) uint64_t tile[kPlaceTile];
  __shared__ int next_big;
  // A thread takes the row at its position in the bucket-ordered member list, not the row of its own index: the
  // lanes of a wave then walk through the same one or two buckets (their loads fall into the same lines instead of
  // 64 lists apart) and write neighbouring slots; only the reads of the row's fitness are scattered.
  for (int t0 = blockIdx.x * blockDim.x; t0 < npad; t0 += gridDim.x * blockDim.x) {
    const int t = t0 + threadIdx.x;
    // Rows of a bucket of more than kPlaceLarge members (thousands of equal rows: a penalty value for every
    // infeasible row, say): the workgroup takes the bucket through LDS, a tile at a time, as composites
    // (key - first key of the bucket) << 32 | row, and every thread counts for its own row: one 64-bit and one 32-bit
    // comparison per member, the members read eight at a time as 16-byte pieces that all lanes share -- a pass over the
    // bucket per workgroup instead of one per thread, each of them a chain of memory round trips (20 000 equal
    // rows: 2.3 ms that way).  (Buckets wider than 2^32 keys keep the walk per thread.)
    int before = 0, smaller = 0;
    bool counted = false;
    int i = 0, b = -1, lo = 0, hi = 0;
    uint64_t ki = 0ull;
    if (t < n) {
      i = members[t];
      ki = member_key[t];
      b = bucket_of(ki, sp);
      lo = start[b];
      hi = start[b + 1];
    }
    if (sp.shift <= 32) {
      const bool big = hi - lo > kPlaceLarge;
      int done_below = -1;  // large buckets up to this one are done (the rows of a workgroup lie in ascending buckets)
      while (__syncthreads_or(big && b > done_below)) {
        __syncthreads();
        if (threadIdx.x == 0) next_big = 0x7FFFFFFF;
        __syncthreads();
        if (big && b > done_below) atomicMin(&next_big, b);
        __syncthreads();
        const int bb = next_big;
        if (bb == 0x7FFFFFFF) break;
        const int blo = start[bb], bhi = start[bb + 1];
        const uint64_t first_key = sp.kmin + ((uint64_t)bb << sp.shift);
        const bool mine = big && b == bb;
        const uint64_t ci = ((ki - first_key) << 32) | (uint32_t)i;
        const uint32_t ci_key = (uint32_t)(ci >> 32);
        for (int p0 = blo; p0 < bhi; p0 += kPlaceTile) {
          __syncthreads();
          for (int e = threadIdx.x; e < kPlaceTile; e += blockDim.x)
            tile[e] = p0 + e < bhi ? ((member_key[p0 + e] - first_key) << 32) | (uint32_t)members[p0 + e] : ~0ull;
          __syncthreads();
          if (mine) {
            for (int e0 = 0; e0 < kPlaceTile; e0 += 8) {
              ulonglong2 c[4];
#pragma unroll
              for (int u = 0; u < 4; ++u) c[u] = *reinterpret_cast<const ulonglong2*>(&tile[e0 + 2 * u]);
#pragma unroll
              for (int u = 0; u < 4; ++u) {
                before += (c[u].x < ci ? 1 : 0) + (c[u].y < ci ? 1 : 0);
                smaller += ((uint32_t)(c[u].x >> 32) < ci_key ? 1 : 0) + ((uint32_t)(c[u].y >> 32) < ci_key ? 1 : 0);
              }
            }
          }
        }
        if (mine) counted = true;
        done_below = bb;
      }
    }
    if (t < n) {
      // eight members at a time, all loads before any use (a bucket of a clustered population holds dozens of rows)
      for (int p0 = counted ? hi : lo; p0 < hi; p0 += 8) {
        int e[8];
        uint64_t ke[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const bool in = p0 + u < hi;
          e[u] = in ? members[p0 + u] : 0x7FFFFFFF;
          ke[u] = in ? member_key[p0 + u] : ~0ull;
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          smaller += ke[u] < ki;
          before += (ke[u] < ki) || (ke[u] == ki && e[u] < i);
        }
      }
      const int slot = lo + before;
      orig_of[slot] = i;
      slot_of[i] = slot;
      key_sorted[slot] = ki;
      kid_sorted[slot] = (uint32_t)(lo + smaller);  // first slot holding this key: equal ids <=> equal keys
      // -0.0 is stored as +0.0: every comparison reads the same, and differences of equal values are +0.0
      for (int k = 0; k < m; ++k) xs_sorted[(int64_t)k * npad + slot] = xs[(int64_t)k * npad + i] + 0.0f;
    } else if (t < npad) {
      orig_of[t] = -1;
      key_sorted[t] = ~0ull;
      kid_sorted[t] = (uint32_t)t;
      for (int k = 0; k < m; ++k) xs_sorted[(int64_t)k * npad + t] = __uint_as_float(0x7FC00000u);
    }
  }
}

}  // namespace evx
