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
//  2. dominance_prefix_kernel: a workgroup takes a tile of 512 dominator slots (8 matrix words, 64 bytes of
//     every row; 256 slots above ten objectives, where the tables of 512 no longer fit the LDS) and a stretch
//     of rows below it.  Restricted to one word of the tile, the prefix of objective k that belongs to row j is
//     one of only 65 bit sets: the word's own slots sorted by pos_k, the first c of them.  The workgroup builds
//     in LDS, per objective: the tile's positions in ascending order (mp), a coarse index from position to the
//     number t of them that lie before it, for every t the byte counts c (how many of the first t fall into each
//     word), and the 65 bit sets of every word, kept complemented.  A lane then needs, per row and objective, one
//     look-up of t (the coarse index, then a comparison or two along mp), one 8-byte read of the counts and one
//     8-byte read of a bit set per word, ORed over the objectives and complemented once: about 55 instructions
//     per objective and 512 pairs, where the pairwise test needs 640.  While it holds the words of a row it also
//     leaves their popcount and the highest non-empty word for the count stage (peel.hpp), which then reads no
//     row again.
#pragma once

#include "common.hpp"
#include "order.hpp"
#include "peel.hpp"
#include "radix.hpp"

namespace evx {

constexpr int kPrefixMaxObjectives = 16;
constexpr int kPrefixWideObjectives = 10;  // up to here tiles of 8 words (14.4 KB of LDS per objective), above it of 4 (9.3 KB)
constexpr int kPrefixBuckets = 1024;       // entries of the coarse index per objective, at most (plus two)
constexpr int kPrefixThreads = 1024;
constexpr int kPrefixRowChunk = 32768;     // rows per workgroup, at most (`chunk`, a multiple of 64)
constexpr int kPrefixMaxRows = 1 << 22;    // a position and a slot of the tile share one int

// LDS of dominance_prefix_kernel<M, WW>, per objective: bit sets and counts (the scratch of the build lies over
// them), sorted positions, the sorted (position, slot) pairs of the build, and the coarse index.
__host__ __device__ inline size_t prefix_lds_bytes(int m, int tile_words, int buckets) {
  const int tile_slots = 64 * tile_words;
  const size_t sets = sizeof(uint64_t) * tile_words * 65;
  const size_t counts = sizeof(uint64_t) * (tile_slots + 1);
  const size_t scratch = (sizeof(int) * (size_t)(buckets + 2 + tile_slots) + 7) & ~(size_t)7;  // histogram, claimed
  const size_t over = sets + counts > scratch ? sets + counts : scratch;
  const size_t positions = sizeof(int) * (tile_slots + 8);
  const size_t sorted = sizeof(int) * tile_slots;
  const size_t index = (sizeof(uint16_t) * (size_t)(buckets + 2) + 7) & ~(size_t)7;
  return (size_t)m * (over + positions + sorted + index);
}

// Positions are cut into at most kPrefixBuckets buckets of 2^shift positions.
__host__ __device__ inline int prefix_bucket_shift(int n) {
  int shift = 0;
  while (((n - 1) >> shift) + 1 > kPrefixBuckets) ++shift;
  return shift;
}

// pos[k * kstride + slot] = position of the slot's row in the ascending order of objective k, equal values in the
// order of the original row index (the order of a stable sort of the population as the caller holds it, which the
// ordering of the last front takes over: front_order_kernels below);
// upper[k * kstride + slot] = number of rows whose value in objective k is at most this slot's.
// `xs` = the fitness by original index, `slot_of` = original index -> slot.  The sorted (key, original index) pairs
// stay in buf.pairs[0] and param->orders_valid says so.
// Grid: the radix grid (all blocks resident).  Dynamic LDS: kRadixLdsBytes.  Nothing is done for a
// population with a NaN or an infinity.
__global__ __launch_bounds__(kRadixThreads) void objective_order_kernel(const float* __restrict__ xs, int npad, int n, int m,
                                                                        const int* __restrict__ slot_of,
                                                                        SortParam* __restrict__ param,
                                                                        Ctrl* __restrict__ ctrl, int* __restrict__ pos,
                                                                        int* __restrict__ upper, int* __restrict__ total0,
                                                                        int* __restrict__ witness0, RadixBuffers buf,
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
  // the row totals that dominance_prefix_kernel accumulates start from nothing
  for (int j = wb * blockDim.x + threadIdx.x; j < n; j += workers * blockDim.x) {
    total0[j] = 0;
    witness0[j] = -1;
  }
  auto initial = [&](int k, int e) { return ((unsigned long long)ordered_key(xs[(int64_t)k * npad + e]) << 32) | (unsigned)e; };
  if (!radix_sort_segments(buf, m, n, initial, ctrl, gen0, spin_limit, order_lds, base, scratch)) return;
  for (int k = 0; k < m; ++k) {
    const unsigned long long* __restrict__ sorted = buf.pairs[0] + (int64_t)k * buf.kstride;
    for (int p = wb * blockDim.x + threadIdx.x; p < n; p += workers * blockDim.x) {
      const unsigned long long pr = coherent_load(&sorted[p]);
      const uint32_t key = (uint32_t)(pr >> 32);
      const int slot = slot_of[(int)(unsigned)(pr & 0xFFFFFFFFull)];
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
  if (wb == 0 && threadIdx.x == 0) param->orders_valid = 1;
}

// The same orders for populations of at most kMidArgsortRows rows, in two launches without a wait between
// workgroups (the radix sort above spends 160 us on its twelve grid barriers whatever the size): the workgroups share
// the objectives out, and each produces a run of positions of its objective's order from all keys of that objective
// in its LDS (mid_argsort_slice); a second kernel derives pos and upper from the sorted pairs.
// Grid: any (one workgroup per compute unit).  Dynamic LDS: mid_sort_lds_bytes(n).
template <bool WIDE>
__global__ __launch_bounds__(kMidArgsortThreads) void objective_order_lds_kernel(const float* __restrict__ xs, int npad, int n, int m,
                                                                                 const SortParam* __restrict__ param,
                                                                                 const Ctrl* __restrict__ ctrl,
                                                                                 int* __restrict__ total0, int* __restrict__ witness0,
                                                                                 RadixBuffers buf) {
  extern __shared__ __attribute__((aligned(16))) uint64_t order_sort_lds[];
  if (param->nonfinite != 0 || ctrl->err != 0) return;
  for (int j = blockIdx.x * blockDim.x + threadIdx.x; j < n; j += gridDim.x * blockDim.x) {
    total0[j] = 0;
    witness0[j] = -1;
  }
  const int nb = (int)gridDim.x;
  const int per_objective = nb >= m ? nb / m : 1;  // workgroups that share an objective
  const int run = ((n + per_objective - 1) / per_objective + 15) & ~15;
  for (int item = blockIdx.x; item < per_objective * m; item += nb) {
    const int k = item % m, s0 = (item / m) * run;
    if (s0 >= n) continue;
    const float* __restrict__ col = xs + (int64_t)k * npad;
    unsigned long long* __restrict__ sorted = buf.pairs[0] + (int64_t)k * buf.kstride;
    mid_argsort_slice<WIDE>(
        order_sort_lds, n, s0, s0 + run, [&](int e) { return ordered_key(col[e]); },
        [&](int p, int e) { sorted[p] = ((unsigned long long)ordered_key(col[e]) << 32) | (unsigned)e; });
  }
}

// The same orders for larger populations, still without a wait between workgroups: the workgroups share the
// objectives out, `parts` to each, and a workgroup produces a run of consecutive positions of its objective's order.
// Rows are composites (key << 20 | original index: distinct, below 2^52).  Every workgroup of an objective sorts the
// same kOrderStreamSample composites (rows n i / sample) and takes the composites between two of them as its share,
// which makes `parts` shares of about n / parts rows whatever the values are, equal ones included; it then reads the
// objective's keys once, counts the composites below its share (where its run starts) and collects those inside it in
// LDS, sorts them there (the bitonic network of radix.hpp over doubles 2^52 + composite, which order like the
// composites) and writes the run.  A share that does not fit `capacity` entries -- rows arranged so that the sample
// misses where they crowd -- is taken in pieces: the largest stretch of composites from the share's start that fits is
// found by bisection over the composites, a pass over the keys per step, as often as it takes.
// Where the time goes (200 000 x 8 in 32 shares of 6250 rows, 154 us): the sort of the sample 23 us, the pass over the
// keys 34 + 20 for storing what it collects, the sort of the share 77 (padded to 8192; 35 when padded to 4096) -- the
// network's passes are what this costs, which is why the host takes this kernel only while shares of at most
// kOrderStreamShare rows leave it no more workgroups than the device has compute units.
// Grid: m * parts workgroups of kOrderStreamThreads.  Dynamic LDS: 8 * kOrderStreamCapacity bytes.  n <= 2^20.
constexpr int kOrderStreamThreads = 1024;
constexpr int kOrderStreamCapacity = 16384;
constexpr int kOrderStreamSample = 2048;
constexpr int kOrderStreamMaxRows = 1 << 20;
constexpr int kOrderStreamShare = 3200;  // rows of a share, at most, that the host aims at: sorted as 4096 entries

__global__ __launch_bounds__(kOrderStreamThreads) void objective_order_stream_kernel(const float* __restrict__ xs, int npad, int n, int m,
                                                                                     int parts, int capacity,
                                                                                     const SortParam* __restrict__ param,
                                                                                     const Ctrl* __restrict__ ctrl,
                                                                                     int* __restrict__ total0, int* __restrict__ witness0,
                                                                                     RadixBuffers buf) {
  extern __shared__ __attribute__((aligned(16))) double order_stream_comp[];
  __shared__ int taken;           // composites of the present pass that lie in its range
  __shared__ int below_of[16];    // per wave: composites below the range
  if (param->nonfinite != 0 || ctrl->err != 0) return;
  for (int j = blockIdx.x * blockDim.x + threadIdx.x; j < n; j += gridDim.x * blockDim.x) {
    total0[j] = 0;
    witness0[j] = -1;
  }
  double* const comp = order_stream_comp;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int k = (int)blockIdx.x % m, part = (int)blockIdx.x / m;
  if (part >= parts) return;
  const float* __restrict__ col = xs + (int64_t)k * npad;
  unsigned long long* __restrict__ sorted = buf.pairs[0] + (int64_t)k * buf.kstride;
  constexpr unsigned long long kBias = 0x4330000000000000ull;  // the bits of 2^52 as a double
  constexpr unsigned long long kEnd = 1ull << 52;               // above every composite
  auto composite = [&](int e) { return ((unsigned long long)ordered_key(col[e]) << 20) | (unsigned long long)(unsigned)e; };

  // ---- the share: between two members of the sorted sample
  for (int i = tid; i < kOrderStreamSample; i += kOrderStreamThreads)
    comp[bitonic_slot(i)] = __longlong_as_double((long long)(kBias | composite((int)(((int64_t)i * n) / kOrderStreamSample))));
  __syncthreads();
  bitonic_sort_lds(comp, kOrderStreamSample);
  auto sample_at = [&](int i) { return (unsigned long long)__double_as_longlong(comp[bitonic_slot(i)]) & (kEnd - 1ull); };
  unsigned long long lo = part == 0 ? 0ull : sample_at((int)(((int64_t)part * kOrderStreamSample) / parts));
  const unsigned long long end = part == parts - 1 ? kEnd : sample_at((int)(((int64_t)(part + 1) * kOrderStreamSample) / parts));
  __syncthreads();  // (the sample is overwritten from here on)

  // One pass over the objective's keys: the composites in [from, to) are counted (the return value) and, with `collect`,
  // the first `capacity` of them stored; *below = the composites smaller than `from`.
  auto pass = [&](unsigned long long from, unsigned long long to, bool collect, int* below) {
    if (tid == 0) taken = 0;
    __syncthreads();
    const unsigned long long span = to - from;
    int under = 0;  // (wave-uniform)
    // (a wave takes 256 keys a step and fetches the keys of kAhead steps before it looks at the first of them)
    constexpr int kAhead = 8;
    for (int g0 = 256 * wave; g0 < n; g0 += kAhead * 4 * kOrderStreamThreads) {  // (wave-uniform)
      float4 q[kAhead];
#pragma unroll
      for (int a = 0; a < kAhead; ++a) {
        const int e0 = g0 + a * 4 * kOrderStreamThreads + 4 * lane;
        q[a] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        if (e0 + 3 < n) {
          q[a] = *reinterpret_cast<const float4*>(col + e0);
        } else if (e0 < n) {
          q[a].x = col[e0];
          if (e0 + 1 < n) q[a].y = col[e0 + 1];
          if (e0 + 2 < n) q[a].z = col[e0 + 2];
        }
      }
#pragma unroll
      for (int a = 0; a < kAhead; ++a) {
        const int b0 = g0 + a * 4 * kOrderStreamThreads;
        if (b0 >= n) break;  // (wave-uniform)
        const int e0 = b0 + 4 * lane;
        const float v[4] = {q[a].x, q[a].y, q[a].z, q[a].w};
        unsigned long long c[4];
        uint64_t in[4];
        int here = 0;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          c[u] = ((unsigned long long)ordered_key(v[u]) << 20) | (unsigned long long)(unsigned)(e0 + u);
          const bool live = e0 + u < n;
          in[u] = __builtin_amdgcn_ballot_w64(live && c[u] - from < span);
          under += __popcll(__builtin_amdgcn_ballot_w64(live && c[u] < from));
          here += __popcll(in[u]);
        }
        if (here != 0) {  // (wave-uniform)
          int at = 0;
          if (lane == 0) at = atomicAdd(&taken, here);
          at = __builtin_amdgcn_readfirstlane(at);
          if (collect) {
#pragma unroll
            for (int u = 0; u < 4; ++u) {
              const int mine = at + __popcll(in[u] & ((1ull << lane) - 1ull));
              if (((in[u] >> lane) & 1ull) != 0ull && mine < capacity)
                comp[bitonic_slot(mine)] = __longlong_as_double((long long)(kBias | c[u]));
              at += __popcll(in[u]);
            }
          }
        }
      }
    }
    if (lane == 0) below_of[wave] = under;
    __syncthreads();
    if (below != nullptr) {
      int sum = 0;
#pragma unroll
      for (int w = 0; w < kOrderStreamThreads / 64; ++w) sum += below_of[w];
      *below = sum;
    }
    const int count = taken;
    __syncthreads();  // (everybody has read the counters before the next pass clears them)
    return count;
  };

  int run_start = 0;
  bool first = true;
  while (lo < end) {  // (the same in every thread)
    unsigned long long hi = end;
    int below = 0;
    int count = pass(lo, hi, true, &below);
    if (first) run_start = below;
    first = false;
    if (count > capacity) {
      // [lo, fits) holds at most one composite; [lo, over) too many
      unsigned long long fits = lo + 1ull, over = hi;
      while (over - fits > 1ull) {
        const unsigned long long mid = fits + (over - fits) / 2ull;
        if (pass(lo, mid, false, nullptr) <= capacity)
          fits = mid;
        else
          over = mid;
      }
      hi = fits;
      count = pass(lo, hi, true, nullptr);
    }
    if (count > 0) {
      int padded = kRowsBitonicMin;
      while (padded < count) padded <<= 1;
      for (int e = count + tid; e < padded; e += kOrderStreamThreads) comp[bitonic_slot(e)] = (double)INFINITY;
      __syncthreads();
      bitonic_sort_lds(comp, padded);
      for (int e = tid; e < count; e += kOrderStreamThreads) {
        const unsigned long long c = (unsigned long long)__double_as_longlong(comp[bitonic_slot(e)]) & (kEnd - 1ull);
        sorted[run_start + e] = ((c >> 20) << 32) | (c & 0xFFFFFull);
      }
      __syncthreads();
    }
    run_start += count;
    lo = hi;
  }
}

__global__ __launch_bounds__(256) void objective_positions_kernel(int n, int m, const int* __restrict__ slot_of,
                                                                  SortParam* __restrict__ param, const Ctrl* __restrict__ ctrl,
                                                                  int* __restrict__ pos, int* __restrict__ upper, RadixBuffers buf) {
  if (param->nonfinite != 0 || ctrl->err != 0) return;
  for (int64_t at = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; at < (int64_t)n * m; at += (int64_t)gridDim.x * blockDim.x) {
    const int k = (int)(at / n), p = (int)(at - (int64_t)k * n);
    const unsigned long long* __restrict__ sorted = buf.pairs[0] + (int64_t)k * buf.kstride;
    const unsigned long long pr = sorted[p];
    const uint32_t key = (uint32_t)(pr >> 32);
    const int slot = slot_of[(int)(unsigned)(pr & 0xFFFFFFFFull)];
    int e = p + 1;
    if (e < n && (uint32_t)(sorted[e] >> 32) == key) {
      // a run of equal values: its end by bisection (the first position whose key is larger, or n)
      int lo = p + 2, hi = n;
      while (lo < hi) {
        const int mid = (lo + hi) >> 1;
        if ((uint32_t)(sorted[mid] >> 32) > key)
          hi = mid;
        else
          lo = mid + 1;
      }
      e = lo;
    }
    pos[(int64_t)k * buf.kstride + slot] = p;
    upper[(int64_t)k * buf.kstride + slot] = e;
  }
  if (blockIdx.x == 0 && threadIdx.x == 0) param->orders_valid = 1;
}

// The value that the neighbouring lane (lane ^ 1) passes in, by two DPP quad permutations.
__device__ inline uint64_t pair_exchange(uint64_t v) {
  const int lo = __builtin_amdgcn_mov_dpp((int)(uint32_t)v, 0xB1, 0xF, 0xF, true);  // quad_perm [1,0,3,2]
  const int hi = __builtin_amdgcn_mov_dpp((int)(uint32_t)(v >> 32), 0xB1, 0xF, 0xF, true);
  return (uint64_t)(uint32_t)lo | ((uint64_t)(uint32_t)hi << 32);
}

// d[2p], d[2p+1] = the p-th 16-byte piece of this lane's row.  Afterwards they hold piece (lane & 3) of the row of
// lane (lane & ~3) + p: the 4 x 4 transpose of the pieces among four neighbouring lanes, in two exchanges (with the
// lane one away, then with the lane two away), every dword moved by one DPP quad permutation.
__device__ inline void quad_transpose_pieces(uint64_t (&d)[8], int lane) {
  int v[16];
#pragma unroll
  for (int w = 0; w < 8; ++w) {
    v[2 * w] = (int)(uint32_t)d[w];
    v[2 * w + 1] = (int)(uint32_t)(d[w] >> 32);
  }
  const bool odd = (lane & 1) != 0, high = (lane & 2) != 0;
  // piece p occupies v[4p .. 4p+3]
#pragma unroll
  for (int h = 0; h < 2; ++h)  // pieces 2h and 2h+1 against the lane one away
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      int& even = v[4 * (2 * h) + x];
      int& oddp = v[4 * (2 * h + 1) + x];
      const int send = odd ? even : oddp;
      const int recv = __builtin_amdgcn_mov_dpp(send, 0xB1, 0xF, 0xF, true);  // quad_perm [1,0,3,2]
      even = odd ? recv : even;
      oddp = odd ? oddp : recv;
    }
#pragma unroll
  for (int h = 0; h < 2; ++h)  // pieces h and h+2 against the lane two away
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      int& low = v[4 * h + x];
      int& hi = v[4 * (h + 2) + x];
      const int send = high ? low : hi;
      const int recv = __builtin_amdgcn_mov_dpp(send, 0x4E, 0xF, 0xF, true);  // quad_perm [2,3,0,1]
      low = high ? recv : low;
      hi = high ? hi : recv;
    }
#pragma unroll
  for (int w = 0; w < 8; ++w) d[w] = (uint64_t)(uint32_t)v[2 * w] | ((uint64_t)(uint32_t)v[2 * w + 1] << 32);
}

// A workgroup takes TT neighbouring tiles of WW words (TT = 2 with WW = 8: the whole 128-byte line of every row).
// grid.x = the ceil(nwords / (WW * TT)) tile groups of dominator slots, rounded up to a multiple of 128 / (WW * TT),
// grid.y = stretches of `chunk` rows, counted from the first row of the tile or (bands) from row 0 (rows above the
// tile have no word there).  Dynamic LDS: TT * prefix_lds_bytes(M, WW, buckets).  Writes the words of its tiles in
// every row of the stretch and adds their popcount to total0[row]; witness0[row] = the highest non-empty word so far
// (both start from objective_order_kernel's 0 and -1).  Sets param->totals_valid.  mode: bit 0 = the row totals,
// bit 1 = the matrix.  unless_front0 (null: always run): the size of front 0, known from a launch with mode 1 and the
// count stage; when it holds `enough` rows nobody will read the matrix, and the launch (mode 2) does nothing.
template <int M, int WW, int TT>
__global__ __launch_bounds__(kPrefixThreads) void dominance_prefix_kernel(const int* __restrict__ pos, const int* __restrict__ upper,
                                                                          const uint32_t* __restrict__ kid,
                                                                          uint64_t* __restrict__ dom, int n, int kstride,
                                                                          int64_t wstride, int nwords, int shift, int buckets,
                                                                          int chunk, int bands, int mode, int* __restrict__ total0,
                                                                          int* __restrict__ witness0, SortParam* __restrict__ param,
                                                                          const int* __restrict__ unless_front0, int enough) {
  constexpr int TS = 64 * WW, T = kPrefixThreads;
  constexpr int TPL = 16 / (WW * TT);  // workgroups that share a 128-byte line of the matrix
  constexpr int MPL = TS / 64;  // members of the tile per lane when a wave walks through them
  extern __shared__ uint64_t prefix_lds[];
  if (param->nonfinite != 0) return;
  if (unless_front0 != nullptr && *unless_front0 >= enough) return;
  if (blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0) param->totals_valid = 1;  // for the count stage
  // Workgroups go to the eight dies in turn (linear index modulo 8), and a die has its own L2.  The tiles
  // that share the 128-byte lines of the matrix are given to consecutive workgroups of one die, which run
  // side by side over the same rows: their pieces of a line then meet in that L2 and leave as one line.
  const int64_t linear = (int64_t)blockIdx.y * gridDim.x + blockIdx.x;
  const int die = (int)(linear & 7);
  const int seq = (int)blockIdx.x >> 3;  // this workgroup among those of its die in this row of the grid
  const int tile = TPL * ((seq / TPL) * 8 + die) + seq % TPL;
  if (tile * WW * TT >= nwords) return;
  const int w0 = tile * WW * TT;  // the first word of the workgroup's TT tiles (tile `sub` starts WW * sub words on)
  const int slot0 = w0 * 64;
  int64_t first_row = (int64_t)slot0 + (int64_t)blockIdx.y * chunk, end_row = first_row + chunk;
  if (bands) {  // the same rows for all tiles of a grid row: the tiles left of the diagonal in rows y * chunk ...
    first_row = (int64_t)blockIdx.y * chunk;
    end_row = first_row + chunk;
    if (first_row < slot0) first_row = slot0;
  }
  if (first_row >= n || first_row >= end_row) return;
  const int r0 = (int)first_row;
  const int r1 = (int)(end_row < n ? end_row : n);
  const int HB = buckets + 2;  // entries of the coarse index per objective
  // per objective k (all arrays [M][...]):
  constexpr int kSetWords = WW * 65;                 // sets[k][w][c]: the slots of the first c members of word w
  constexpr int kOver = kSetWords + TS + 1;          // ... then counts[k][t]: eight byte counts, members of each word among the first t
  const int scratch_words = (HB + TS + 1) / 2;       // histogram and claimed pairs of the build, in the same place
  const int over = kOver > scratch_words ? kOver : scratch_words;
  // the tables of tile `sub` of the workgroup (TT = 2: the two tiles of a 128-byte line, so that the workgroup writes
  // whole lines; their tables fit the LDS up to four objectives)
  const size_t tile_lds_words = prefix_lds_bytes(M, WW, buckets) / sizeof(uint64_t);
  uint64_t* tile_lds = prefix_lds;
  uint64_t* sets = nullptr;
  uint64_t* counts = nullptr;
  int* mp = nullptr;           // [M][TS + 8]: positions ascending, then INT_MAX
  int* sorted = nullptr;       // [M][TS]: position << 9 | slot in tile, ascending
  uint16_t* index = nullptr;   // [M][HB]: members in earlier buckets
  int live = 0;                // slots of the tile that hold a row
  int tile_slot0 = slot0;
  auto select_tile = [&](int sub) {
    tile_lds = prefix_lds + (size_t)sub * tile_lds_words;
    sets = tile_lds;
    counts = sets + kSetWords;
    mp = reinterpret_cast<int*>(tile_lds + (size_t)M * over);
    sorted = mp + M * (TS + 8);
    index = reinterpret_cast<uint16_t*>(sorted + M * TS);
    tile_slot0 = slot0 + sub * TS;
    live = n - tile_slot0 < TS ? n - tile_slot0 : TS;
  };
  auto hist_of = [&](int k) { return reinterpret_cast<int*>(tile_lds + (size_t)k * over); };  // [HB]
  auto claimed_of = [&](int k) { return hist_of(k) + HB; };                                      // [TS]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int index_stride = (HB + 3) & ~3;

  for (int sub = 0; sub < TT; ++sub) {
  select_tile(sub);
  // ---- the tile's slots by position, objective by objective
  for (int t = threadIdx.x; t < M * HB; t += T) hist_of(t / HB)[t % HB] = 0;
  for (int t = threadIdx.x; t < M * (TS + 8); t += T) mp[t] = 0x7FFFFFFF;
  __syncthreads();
  constexpr int PER = (M * TS + T - 1) / T;
  int mine[PER];
#pragma unroll
  for (int u = 0; u < PER; ++u) {
    const int item = threadIdx.x + u * T;
    const int k = item / TS, i = item - k * TS;
    mine[u] = -1;
    if (item < M * TS && i < live) {
      const int p = pos[(int64_t)k * kstride + tile_slot0 + i];
      mine[u] = (p << 9) | i;
      atomicAdd(&hist_of(k)[p >> shift], 1);
    }
  }
  __syncthreads();
  if (wave < M) {  // exclusive prefix of the bucket counts of objective `wave`
    int carry = 0;
    for (int b0 = 0; b0 < HB; b0 += 64) {
      const int b = b0 + lane;
      const int v = b < HB ? hist_of(wave)[b] : 0;
      int incl = v;
#pragma unroll
      for (int off = 1; off < 64; off <<= 1) {
        const int up = __shfl_up(incl, off);
        if (lane >= off) incl += up;
      }
      if (b < HB) index[wave * index_stride + b] = (uint16_t)(carry + incl - v);
      carry += __shfl(incl, 63);
    }
  }
  __syncthreads();
#pragma unroll
  for (int u = 0; u < PER; ++u) {
    if (mine[u] >= 0) {
      const int k = (threadIdx.x + u * T) / TS;
      const int b = (mine[u] >> 9) >> shift;
      const int r = atomicSub(&hist_of(k)[b], 1) - 1;
      claimed_of(k)[(int)index[k * index_stride + b] + r] = mine[u];
    }
  }
  __syncthreads();
#pragma unroll
  for (int u = 0; u < PER; ++u) {
    if (mine[u] >= 0) {
      const int k = (threadIdx.x + u * T) / TS;
      const int b = (mine[u] >> 9) >> shift;
      const int t0 = index[k * index_stride + b], t1 = index[k * index_stride + b + 1];
      int before = 0;
      for (int t = t0; t < t1; ++t) before += claimed_of(k)[t] < mine[u] ? 1 : 0;
      sorted[k * TS + t0 + before] = mine[u];
      mp[k * (TS + 8) + t0 + before] = mine[u] >> 9;
    }
  }
  __syncthreads();
  // ---- counts[k][t] and the single bits of sets[k][w][c + 1]; a wave per objective, a lane per MPL members
  for (int t = threadIdx.x; t < M * kSetWords; t += T) sets[(size_t)(t / kSetWords) * over + t % kSetWords] = 0ull;
  __syncthreads();
  for (int k = wave; k < M; k += T / 64) {
    uint64_t one[MPL];
    uint64_t sum = 0ull;
#pragma unroll
    for (int c = 0; c < MPL; ++c) {
      const int t = MPL * lane + c;
      one[c] = t < live ? 1ull << (8 * ((sorted[k * TS + t] & (TS - 1)) >> 6)) : 0ull;
      sum += one[c];
    }
    uint64_t incl = sum;  // byte-wise counts: at most 64 per byte, no carry between bytes
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const uint64_t up = __shfl_up(incl, off);
      if (lane >= off) incl += up;
    }
    uint64_t run = incl - sum;  // members before this lane's eight
    uint64_t* const cnt = counts + (size_t)k * over;
    uint64_t* const set = sets + (size_t)k * over;
#pragma unroll
    for (int c = 0; c < MPL; ++c) {
      const int t = MPL * lane + c;
      cnt[t] = run;
      if (t < live) {
        const int i = sorted[k * TS + t] & (TS - 1);
        const int w = i >> 6;
        const int rank_in_word = (int)((run >> (8 * w)) & 255ull);
        set[w * 65 + rank_in_word + 1] = 1ull << (i & 63);
      }
      run += one[c];
    }
    if (lane == 63) cnt[TS] = run;
  }
  __syncthreads();
  // ---- sets[k][w][c] = OR of the single bits up to c; a wave per (objective, word)
  for (int item = wave; item < M * WW; item += T / 64) {
    const int k = item / WW, w = item - k * WW;
    uint64_t* const col = sets + (size_t)k * over + w * 65;
    uint64_t incl = col[lane + 1];
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const uint64_t up = __shfl_up(incl, off);
      if (lane >= off) incl |= up;
    }
    col[lane + 1] = ~incl;  // kept complemented: a row ORs the complements of its M sets (three-input ORs) and
    if (lane == 0) col[0] = ~0ull;  // complements once
  }
  __syncthreads();

  }  // tiles of the workgroup

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
    uint64_t dd[TT][WW];  // per tile: slots that are worse than row j in some objective, then its dominators
    int dominators = 0, highest = -1;
#pragma unroll
    for (int sub = 0; sub < TT; ++sub) {
      select_tile(sub);
      const int tw0 = w0 + sub * WW;
      uint64_t(&d)[WW] = dd[sub];
      // t[k] = members of objective k that lie before upper_k(j): those of the earlier buckets plus those of the
      // bucket itself that do (positions ascend, so the members from t on that lie before it are consecutive)
      int t[M];
      bool more = false;
#pragma unroll
      for (int k = 0; k < M; ++k) t[k] = index[k * index_stride + (e[k] >> shift)];
#pragma unroll
      for (int k = 0; k < M; ++k) {
        const int m0 = mp[k * (TS + 8) + t[k]], m1 = mp[k * (TS + 8) + t[k] + 1];
        const int a0 = m0 < e[k] ? 1 : 0, a1 = m1 < e[k] ? 1 : 0;
        t[k] += a0 + a1;
        more |= a1 != 0;
      }
      if (__builtin_amdgcn_ballot_w64(more) != 0ull) {  // three or more members of the tile in one bucket: rare
#pragma unroll
        for (int k = 0; k < M; ++k)
          while (mp[k * (TS + 8) + t[k]] < e[k]) ++t[k];
      }
#pragma unroll
      for (int w = 0; w < WW; ++w) d[w] = 0ull;
#pragma unroll
      for (int k = 0; k < M; ++k) {
        const uint64_t c8 = counts[(size_t)k * over + t[k]];
        const uint64_t* const set = sets + (size_t)k * over;
#pragma unroll
        for (int w = 0; w < WW; ++w) d[w] |= set[w * 65 + (int)((c8 >> (8 * w)) & 255ull)];
      }
#pragma unroll
      for (int w = 0; w < WW; ++w) d[w] = ~d[w];
      // rows identical to j and everything after them: only near the diagonal (wave-uniform test)
      if (__builtin_amdgcn_ballot_w64(same_from < tile_slot0 + TS) != 0ull) {
#pragma unroll
        for (int w = 0; w < WW; ++w) {
          const int first = (tw0 + w) * 64;
          if (same_from <= first)
            d[w] = 0ull;
          else if (same_from < first + 64)
            d[w] &= (1ull << (same_from - first)) - 1ull;
        }
      }
      // what the count stage wants to know of the row, so that it does not have to read it again
#pragma unroll
      for (int w = 0; w < WW; ++w) {
        dominators += __popcll(d[w]);
        highest = d[w] != 0ull ? tw0 + w : highest;
      }
    }
    if (j < n && (mode & 1) && dominators != 0) {
      atomicAdd(&total0[j], dominators);
      atomicMax(&witness0[j], highest);
    }
    if (!(mode & 2)) continue;
    if constexpr (WW == 8 && TT == 2) {
      // Eight neighbouring lanes transpose the eight 16-byte pieces of their rows' lines (four of each tile): inside
      // the quads as below, then the lower quad hands its pieces of the second tile to the upper quad for the upper
      // quad's pieces of the first.  A store instruction then writes the whole 128-byte line of a row from eight
      // lanes side by side: one request of a line to memory instead of two of half a line.
      quad_transpose_pieces(dd[0], lane);
      quad_transpose_pieces(dd[1], lane);
      const bool upper_quad = (lane & 4) != 0;
      uint64_t other[8];  // piece (lane & 7) of the rows of the other quad
#pragma unroll
      for (int x = 0; x < 8; ++x) {
        const uint64_t send = upper_quad ? dd[0][x] : dd[1][x];
        const int lo = __shfl_xor((int)(uint32_t)send, 4);
        const int hi = __shfl_xor((int)(uint32_t)(send >> 32), 4);
        other[x] = (uint64_t)(uint32_t)lo | ((uint64_t)(uint32_t)hi << 32);
      }
      const int j8 = j - (lane & 7);  // the first row of this lane's eight
#pragma unroll
      for (int p = 0; p < 8; ++p) {
        // rows 0..3 of the eight belong to the lower quad, rows 4..7 to the upper one
        const int q = p & 3;
        const bool own = (p >= 4) == upper_quad;
        const uint64_t a = own ? (upper_quad ? dd[1][2 * q] : dd[0][2 * q]) : other[2 * q];
        const uint64_t b = own ? (upper_quad ? dd[1][2 * q + 1] : dd[0][2 * q + 1]) : other[2 * q + 1];
        if (j8 + p < n)
          *reinterpret_cast<ulonglong2*>(dom + (int64_t)(j8 + p) * wstride + w0 + 2 * (lane & 7)) = make_ulonglong2(a, b);
      }
      continue;
    }
#pragma unroll
    for (int sub = 0; sub < TT; ++sub) {
      const int tw0 = w0 + sub * WW;
      uint64_t(&d)[WW] = dd[sub];
      if constexpr (WW == 8) {
        // Four neighbouring lanes exchange their 16-byte pieces (a 4 x 4 transpose through DPP moves), so that a
        // store instruction writes the whole 64 bytes of a row from four lanes side by side -- one request per row
        // to the memory system instead of four requests of 16 bytes from four instructions.  With two tiles per
        // workgroup the two halves of a row's line follow one another and leave the cache as one line.
        quad_transpose_pieces(d, lane);
        const int jq = j - (lane & 3);  // the first row of this lane's four
#pragma unroll
        for (int p = 0; p < 4; ++p)
          if (jq + p < n)
            *reinterpret_cast<ulonglong2*>(dom + (int64_t)(jq + p) * wstride + tw0 + 2 * (lane & 3)) =
                make_ulonglong2(d[2 * p], d[2 * p + 1]);
      } else {
        // tiles of four words: two neighbouring lanes exchange one piece each, a store writes the 32 bytes of a row
        static_assert(WW == 4, "tiles of four or eight words");
        const bool odd = (lane & 1) != 0;
        const uint64_t s0 = odd ? d[0] : d[2], s1 = odd ? d[1] : d[3];
        const uint64_t g0 = pair_exchange(s0), g1 = pair_exchange(s1);
        const uint64_t a0 = odd ? g0 : d[0], a1 = odd ? g1 : d[1];  // piece (lane & 1) of the even lane's row
        const uint64_t b0 = odd ? d[2] : g0, b1 = odd ? d[3] : g1;  // piece (lane & 1) of the odd lane's row
        const int jp = j - (lane & 1);
        if (jp < n) *reinterpret_cast<ulonglong2*>(dom + (int64_t)jp * wstride + tw0 + 2 * (lane & 1)) = make_ulonglong2(a0, a1);
        if (jp + 1 < n)
          *reinterpret_cast<ulonglong2*>(dom + (int64_t)(jp + 1) * wstride + tw0 + 2 * (lane & 1)) = make_ulonglong2(b0, b1);
      }
    }
  }
}

}  // namespace evx
