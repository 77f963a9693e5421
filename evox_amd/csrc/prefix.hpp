// The dominance bit matrix of a large finite population without testing pair by pair.
//
// Same matrix as dominance.hpp (src/evox/operators/selection/non_dominate.py:6-26 in slot space, lower
// triangle), from the order of the rows in each objective.  With pos_k(i) = position of row i in the
// ascending order of objective k and upper_k(j) = number of rows whose value in objective k is at most row j's,
//     x[i,k] <= x[j,k]  <=>  pos_k(i) < upper_k(j),
// so the rows that are no worse than j in objective k are a prefix of that order, and the dominators of j are
// the intersection over k of the M prefixes, less the rows identical to j (kid(i) == kid(j): equal in every
// objective; a row of a larger slot has a larger key sum and is never in the intersection).  Infinities and
// NaN are left to the pairwise kernel (a NaN has no place in the order).
//
//  1. objective_order_kernel: one segmented radix sort orders the slots by every objective (radix.hpp) and
//     leaves pos[k][slot] and upper[k][slot].
//  2. dominance_prefix_kernel: a workgroup takes a tile of kPrefixTileSlots dominator slots (4 matrix words)
//     and a stretch of rows below it.  Restricted to the tile, the prefix of objective k that belongs to row j
//     is one of only 257 bit sets: the tile's own slots sorted by pos_k, the first t of them, where
//     t = how many of them lie before upper_k(j).  The workgroup builds these tables in LDS (8 KB per
//     objective) together with a coarse index from position to t; a lane then needs, per row and objective, one
//     look-up of t (the coarse index, then a step or two along the tile's sorted positions) and one 32-byte read
//     of the bit set, ANDed over the objectives: about 20 instructions per objective and 256 pairs, where the
//     pairwise test needs 320.
#pragma once

#include "common.hpp"
#include "order.hpp"
#include "peel.hpp"
#include "radix.hpp"

namespace evx {

constexpr int kPrefixTileWords = 4;
constexpr int kPrefixTileSlots = 64 * kPrefixTileWords;
constexpr int kPrefixMaxObjectives = 8;   // 8224 bytes of bit sets per objective
constexpr int kPrefixBuckets = 512;       // entries of the coarse index per objective, at most (plus two)
constexpr int kPrefixThreads = 1024;
constexpr int kPrefixRowChunk = 32768;    // rows per workgroup, at most (`chunk`, a multiple of 64)
constexpr int kPrefixMaxRows = 1 << 22;   // a position and a slot of the tile share one int

// LDS of dominance_prefix_kernel<M>.
__host__ __device__ inline size_t prefix_lds_bytes(int m, int buckets) {
  const size_t sets = sizeof(uint64_t) * (size_t)m * (kPrefixTileSlots + 1) * kPrefixTileWords;  // also the histogram
  const size_t members = sizeof(int) * (size_t)m * kPrefixTileSlots * 2;
  const size_t index = (sizeof(uint32_t) * (size_t)m * (buckets + 2) + 15) & ~(size_t)15;
  return sets + members + index;
}

// Positions are cut into at most kPrefixBuckets buckets of 2^shift positions.
__host__ __device__ inline int prefix_bucket_shift(int n) {
  int shift = 0;
  while (((n - 1) >> shift) + 1 > kPrefixBuckets) ++shift;
  return shift;
}

// pos[k * kstride + slot] = position of the slot in the ascending order of objective k (ties in any order);
// upper[k * kstride + slot] = number of slots whose value in objective k is at most this slot's.
// Grid: the radix grid (all blocks resident).  Dynamic LDS: m * 4 * 256 ints.  Nothing is done for a
// population with a NaN or an infinity.
__global__ __launch_bounds__(kRadixThreads) void objective_order_kernel(const float* __restrict__ xs, int npad, int n, int m,
                                                                        const SortParam* __restrict__ param,
                                                                        Ctrl* __restrict__ ctrl, int* __restrict__ pos,
                                                                        int* __restrict__ upper, RadixBuffers buf,
                                                                        unsigned spin_limit) {
  extern __shared__ int order_lds[];
  __shared__ int base[256];
  __shared__ int scratch[kRadixThreads];
  if (param->nonfinite != 0) return;
  if (coherent_load(&ctrl->err) != 0) return;
  const unsigned gen0 = radix_generation_base(ctrl);
  if (blockIdx.x == 0) {
    radix_master(ctrl, gen0, 12, spin_limit, scratch);
    if (threadIdx.x == 0) ctrl->radix_epoch += 1;  // nobody reads it again in this kernel
    return;
  }
  if (blockIdx.x < kFirstSweeper) return;
  const int workers = gridDim.x - kFirstSweeper;
  const int wb = (int)blockIdx.x - kFirstSweeper;
  auto initial = [&](int k, int e) { return ((unsigned long long)ordered_key(xs[(int64_t)k * npad + e]) << 32) | (unsigned)e; };
  if (!radix_sort_segments(buf, m, n, initial, ctrl, gen0, spin_limit, order_lds, base, scratch)) return;
  for (int k = 0; k < m; ++k) {
    const unsigned long long* __restrict__ sorted = buf.pairs[0] + (int64_t)k * buf.kstride;
    for (int p = wb * blockDim.x + threadIdx.x; p < n; p += workers * blockDim.x) {
      const unsigned long long pr = coherent_load(&sorted[p]);
      const uint32_t key = (uint32_t)(pr >> 32);
      const int slot = (int)(unsigned)(pr & 0xFFFFFFFFull);
      int e = p + 1;
      if (e < n && (uint32_t)(coherent_load(&sorted[e]) >> 32) == key) {
        // a run of equal values: its end by bisection (the first position whose key is larger, or n)
        int lo = p + 2, hi = n;
        while (lo < hi) {
          const int mid = (lo + hi) >> 1;
          if ((uint32_t)(coherent_load(&sorted[mid]) >> 32) > key)
            hi = mid;
          else
            lo = mid + 1;
        }
        e = lo;
      }
      pos[(int64_t)k * buf.kstride + slot] = p;
      upper[(int64_t)k * buf.kstride + slot] = e;
    }
  }
}

// grid.x = the ceil(nwords / kPrefixTileWords) tiles of dominator slots, rounded up to a multiple of 32,
// grid.y = stretches of `chunk` rows, counted from the first row of the tile (rows above it have no
// word there).  Dynamic LDS:
// prefix_lds_bytes(M, buckets).  Writes words 4 * blockIdx.x .. + 3 of every row of the stretch.
template <int M>
__global__ __launch_bounds__(kPrefixThreads) void dominance_prefix_kernel(const int* __restrict__ pos, const int* __restrict__ upper,
                                                                          const uint32_t* __restrict__ kid,
                                                                          uint64_t* __restrict__ dom, int n, int kstride,
                                                                          int64_t wstride, int nwords, int shift, int buckets,
                                                                          int chunk, const SortParam* __restrict__ param) {
  constexpr int WW = kPrefixTileWords, TS = kPrefixTileSlots, T = kPrefixThreads;
  extern __shared__ uint64_t prefix_lds[];
  if (param->nonfinite != 0) return;
  // Workgroups go to the eight dies in turn (linear index modulo 8), and a die has its own L2.  The four tiles
  // that share the 128-byte lines of the matrix are given to consecutive workgroups of one die, which run
  // side by side over the same rows: their 32-byte pieces of a line then meet in that L2 and leave as one line.
  const int64_t linear = (int64_t)blockIdx.y * gridDim.x + blockIdx.x;
  const int die = (int)(linear & 7);
  const int seq = (int)blockIdx.x >> 3;  // this workgroup among those of its die in this row of the grid
  const int tile = 4 * ((seq >> 2) * 8 + die) + (seq & 3);
  if (tile * WW >= nwords) return;
  const int w0 = tile * WW;
  const int slot0 = w0 * 64;
  const int64_t first_row = (int64_t)slot0 + (int64_t)blockIdx.y * chunk;
  if (first_row >= n) return;
  const int r0 = (int)first_row;
  const int r1 = (int)(first_row + chunk < n ? first_row + chunk : n);
  const int HB = buckets + 2;  // entries of the coarse index per objective
  uint64_t* const sets = prefix_lds;                                          // [M][TS + 1][WW]
  int* const hist = reinterpret_cast<int*>(sets);                             // [M][HB] while the tables are built
  int* const member = reinterpret_cast<int*>(sets + (size_t)M * (TS + 1) * WW);  // [M][TS]: position << 8 | slot in tile, ascending
  int* const claimed = member + M * TS;                                       // [M][TS]: the same, unordered inside a bucket
  uint32_t* const index = reinterpret_cast<uint32_t*>(claimed + M * TS);      // [M][HB]: members before the bucket | members in it << 16
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int live = n - slot0 < TS ? n - slot0 : TS;  // slots of the tile that hold a row

  // ---- the tile's slots by position, objective by objective
  for (int t = threadIdx.x; t < M * HB; t += T) hist[t] = 0;
  __syncthreads();
  constexpr int PER = (M * TS + T - 1) / T;
  int mine[PER];
#pragma unroll
  for (int u = 0; u < PER; ++u) {
    const int item = threadIdx.x + u * T;
    const int k = item / TS, i = item - k * TS;
    mine[u] = -1;
    if (item < M * TS && i < live) {
      const int p = pos[(int64_t)k * kstride + slot0 + i];
      mine[u] = (p << 8) | i;
      atomicAdd(&hist[k * HB + (p >> shift)], 1);
    }
  }
  __syncthreads();
  if (wave < M) {  // exclusive prefix of the bucket counts of objective `wave`
    int carry = 0;
    for (int b0 = 0; b0 < HB; b0 += 64) {
      const int b = b0 + lane;
      const int v = b < HB ? hist[wave * HB + b] : 0;
      int incl = v;
#pragma unroll
      for (int off = 1; off < 64; off <<= 1) {
        const int up = __shfl_up(incl, off);
        if (lane >= off) incl += up;
      }
      if (b < HB) index[wave * HB + b] = (uint32_t)(carry + incl - v) | ((uint32_t)v << 16);
      carry += __shfl(incl, 63);
    }
  }
  __syncthreads();
#pragma unroll
  for (int u = 0; u < PER; ++u) {
    if (mine[u] >= 0) {
      const int k = (threadIdx.x + u * T) / TS;
      const int b = (mine[u] >> 8) >> shift;
      const int r = atomicSub(&hist[k * HB + b], 1) - 1;
      claimed[k * TS + (int)(index[k * HB + b] & 0xFFFFu) + r] = mine[u];
    }
  }
  __syncthreads();
#pragma unroll
  for (int u = 0; u < PER; ++u) {
    if (mine[u] >= 0) {
      const int k = (threadIdx.x + u * T) / TS;
      const int b = (mine[u] >> 8) >> shift;
      const uint32_t entry = index[k * HB + b];
      const int t0 = (int)(entry & 0xFFFFu), t1 = t0 + (int)(entry >> 16);
      int before = 0;
      for (int t = t0; t < t1; ++t) before += claimed[k * TS + t] < mine[u] ? 1 : 0;
      member[k * TS + t0 + before] = mine[u];
    }
  }
  __syncthreads();
  // ---- sets[k][t] = the slots of the first t members of objective k; a wave per (objective, word)
  for (int item = wave; item < M * WW; item += T / 64) {
    const int k = item / WW, w = item - k * WW;
    uint64_t bits[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int t = 4 * lane + c;
      const int ent = t < live ? member[k * TS + t] : -1;
      const int i = ent & 255;
      bits[c] = (ent >= 0 && (i >> 6) == w) ? 1ull << (i & 63) : 0ull;
    }
    const uint64_t b0 = bits[0], b1 = b0 | bits[1], b2 = b1 | bits[2], b3 = b2 | bits[3];
    uint64_t incl = b3;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const uint64_t up = __shfl_up(incl, off);
      if (lane >= off) incl |= up;
    }
    uint64_t excl = __shfl_up(incl, 1);
    if (lane == 0) excl = 0ull;
    uint64_t* const col = sets + (size_t)k * (TS + 1) * WW + w;
    col[(size_t)(4 * lane + 0) * WW] = excl;
    col[(size_t)(4 * lane + 1) * WW] = excl | b0;
    col[(size_t)(4 * lane + 2) * WW] = excl | b1;
    col[(size_t)(4 * lane + 3) * WW] = excl | b2;
    if (lane == 63) col[(size_t)TS * WW] = excl | b3;
  }
  __syncthreads();

  // ---- the rows of the stretch, 64 at a time per wave; the inputs of a wave's next rows are fetched while it
  // works on the present ones
  const int groups = (r1 - r0 + 63) / 64;
  int e_next[M];
  int same_next = 0;
  auto fetch = [&](int g) {
    const int j = r0 + g * 64 + lane;
    const int jc = j < n ? j : n - 1;
#pragma unroll
    for (int k = 0; k < M; ++k) e_next[k] = upper[(int64_t)k * kstride + jc];
    same_next = (int)kid[jc];
  };
  if (wave < groups) fetch(wave);
  for (int g = wave; g < groups; g += T / 64) {
    const int j = r0 + g * 64 + lane;
    int e[M];
#pragma unroll
    for (int k = 0; k < M; ++k) e[k] = e_next[k];
    const int same_from = same_next;  // slots from here on hold rows with the key of row j, or larger keys
    if (g + T / 64 < groups) fetch(g + T / 64);
    // t[k] = members of objective k that lie before upper_k(j): those of the earlier buckets, then a step or
    // two inside the bucket (the look-ups of all objectives are in flight together)
    int t[M], t1[M];
#pragma unroll
    for (int k = 0; k < M; ++k) {
      const uint32_t entry = index[k * HB + (e[k] >> shift)];
      t[k] = (int)(entry & 0xFFFFu);
      t1[k] = t[k] + (int)(entry >> 16);
    }
    bool more = false;
#pragma unroll
    for (int step = 0; step < 2; ++step) {
      int first[M];
#pragma unroll
      for (int k = 0; k < M; ++k) first[k] = member[k * TS + (t[k] < TS ? t[k] : TS - 1)];
#pragma unroll
      for (int k = 0; k < M; ++k) {
        const bool advance = t[k] < t1[k] && (first[k] >> 8) < e[k];
        t[k] += advance ? 1 : 0;
        if (step == 1) more |= advance && t[k] < t1[k];
      }
    }
    if (__builtin_amdgcn_ballot_w64(more) != 0ull) {  // a bucket with three or more members of the tile: rare
#pragma unroll
      for (int k = 0; k < M; ++k)
        while (t[k] < t1[k] && (member[k * TS + t[k]] >> 8) < e[k]) ++t[k];
    }
    uint64_t d[WW];
    {
      ulonglong2 lo[M], hi[M];
#pragma unroll
      for (int k = 0; k < M; ++k) {
        const ulonglong2* const set = reinterpret_cast<const ulonglong2*>(sets + ((size_t)k * (TS + 1) + t[k]) * WW);
        lo[k] = set[0];
        hi[k] = set[1];
      }
      d[0] = lo[0].x;
      d[1] = lo[0].y;
      d[2] = hi[0].x;
      d[3] = hi[0].y;
#pragma unroll
      for (int k = 1; k < M; ++k) {
        d[0] &= lo[k].x;
        d[1] &= lo[k].y;
        d[2] &= hi[k].x;
        d[3] &= hi[k].y;
      }
    }
#pragma unroll
    for (int w = 0; w < WW; ++w) {
      const int first = (w0 + w) * 64;
      if (same_from <= first)
        d[w] = 0ull;
      else if (same_from < first + 64)
        d[w] &= (1ull << (same_from - first)) - 1ull;
    }
    if (j < n) {
      ulonglong2* const out = reinterpret_cast<ulonglong2*>(dom + (int64_t)j * wstride + w0);
      out[0] = make_ulonglong2(d[0], d[1]);
      out[1] = make_ulonglong2(d[2], d[3]);
    }
  }
}

}  // namespace evx
