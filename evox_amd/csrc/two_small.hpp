// Two objectives, up to 4096 rows, one workgroup per population, no dominance matrix.
//
// Reference semantics: non_dominate_rank (src/evox/operators/selection/non_dominate.py:172-195, batched :107-125),
// crowding_distance (:198-231) and nd_environmental_selection (:234-254) for M = 2.
//
// With the rows in the order of (f1, f2, index), a row is dominated exactly by the earlier rows whose f2 is smaller
// or equal and that are not copies of it, so front r is the set of strict prefix minima of f2 among the rows that
// fronts 0 .. r-1 have left (two.hpp does the same across workgroups for large populations).  Two objectives mean
// many thin fronts (C2: 20 fronts of 100 rows), which cost the matrix kernels an exchange between workgroups each;
// here a front is one prefix minimum over registers, sixteen wave results through LDS and one barrier.
//
// Everything is a stable LSD radix sort of (32-bit key, 16-bit payload) pairs in LDS, eight bits a pass:
//   * the order of (f1, f2, index): four passes on the key of f1 (ordered_key, common.hpp) where no two rows share an
//     f1, else four on the key of f2 and four on that of f1;
//   * the listing of the fronts by (rank, index): one or two passes on the ranks;
//   * the last front: its rows by each objective for the crowding distances and by the distance for the index-stable
//     top-k -- by counting while it has at most 1024 rows, by the radix sort above.
// A pass ranks the items of a wave among those of equal digit with eight ballots a row of 64 items (stable, no
// atomics), keeps a counter per (digit, wave) and scans the 4096 counters once.
#pragma once

#include "batched.hpp"
#include "peel.hpp"
#include "two.hpp"

// Hook for timing builds; nothing otherwise.
#ifndef EVX_PASS_TRACE
#define EVX_PASS_TRACE(slot)
#endif

namespace evx {

constexpr int kTwoSmallThreads = 1024;
constexpr int kTwoSmallRows = 4096;
constexpr int kTwoSmallPer = kTwoSmallRows / kTwoSmallThreads;  // items of a thread in every pass
constexpr int kTwoSmallCounting = 1024;  // last fronts of at most this many rows are ordered by counting
constexpr uint16_t kTwoSmallUnset = 0xFFFFu;
// dynamic LDS: keys and payloads of the sort twice over, its counters, the keys of both objectives by row, ranks,
// the three orders, the distances
constexpr size_t kTwoSmallLdsBytes = (size_t)kTwoSmallRows * (4 + 4 + 2 + 2 + 4 + 4 + 4 + 2 + 2 + 2 + 2 + 4);

// Inclusive prefix sum over the lanes of a wave (DPP row shifts and row broadcasts, as wave_prefix_min).
__device__ inline uint32_t wave_prefix_sum(uint32_t x) {
  uint32_t v = x;
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x111, 0xf, 0xf, false);  // row_shr:1
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x112, 0xf, 0xf, false);  // row_shr:2
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x113, 0xf, 0xf, false);  // row_shr:3
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x114, 0xf, 0xe, false);  // row_shr:4
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x118, 0xf, 0xc, false);  // row_shr:8
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x142, 0xa, 0xf, false);  // row_bcast:15
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x143, 0xc, 0xf, false);  // row_bcast:31
  return v;
}

// The sum, minimum or maximum of words 0 .. wave-1 of sixteen words in LDS, the same in every lane: lane i < wave
// takes word i, four DPP steps fold the first row of sixteen lanes, and its last lane holds the result.  (Every vector
// instruction of a workgroup of sixteen waves costs the compute unit sixteen issue slots; a fold written as sixteen
// selects and additions per lane was a third of a round of the peeling.)
__device__ inline uint32_t sum_before_wave(const uint32_t* sixteen, int wave) {
  const int lane = threadIdx.x & 63;
  int v = lane < wave ? (int)sixteen[lane & 15] : 0;
  v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, true);  // row_shr:1
  v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, true);  // row_shr:2
  v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xe, true);  // row_shr:4
  v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xc, true);  // row_shr:8
  return (uint32_t)__builtin_amdgcn_readlane(v, 15);
}
__device__ inline uint32_t min_before_wave(const uint32_t* sixteen, int wave) {
  const int lane = threadIdx.x & 63;
  uint32_t v = lane < wave ? sixteen[lane & 15] : kTwoNone;
  v = min(v, (uint32_t)__builtin_amdgcn_update_dpp((int)kTwoNone, (int)v, 0x111, 0xf, 0xf, false));
  v = min(v, (uint32_t)__builtin_amdgcn_update_dpp((int)kTwoNone, (int)v, 0x112, 0xf, 0xf, false));
  v = min(v, (uint32_t)__builtin_amdgcn_update_dpp((int)kTwoNone, (int)v, 0x114, 0xf, 0xe, false));
  v = min(v, (uint32_t)__builtin_amdgcn_update_dpp((int)kTwoNone, (int)v, 0x118, 0xf, 0xc, false));
  return (uint32_t)__builtin_amdgcn_readlane((int)v, 15);
}
__device__ inline uint32_t max_before_wave(const uint32_t* sixteen, int wave) {
  const int lane = threadIdx.x & 63;
  uint32_t v = lane < wave ? sixteen[lane & 15] : 0u;
  v = max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x111, 0xf, 0xf, false));
  v = max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x112, 0xf, 0xf, false));
  v = max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x114, 0xf, 0xe, false));
  v = max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x118, 0xf, 0xc, false));
  return (uint32_t)__builtin_amdgcn_readlane((int)v, 15);
}

// One stable pass of the sort: items 0 .. count-1 of (key_in, pay_in) go to (key_out, pay_out) in the order of the
// digit (key >> shift) & 255, items of equal digit in the order they had.  Called by all kTwoSmallThreads threads.
// cnt: 4096 counters (wave * 256 + digit); part: 16 words; lanes_a: 16 KB of LDS that is free during the pass (with
// key_out, which is written only at the end: a table of 256 lane masks per wave).  Ends with a barrier.
//   1. every wave counts its items per digit, row by row (64 items): every lane sets its bit in the wave's table entry
//      of its digit (an LDS atomic) and reads the entry back -- the lanes of equal digit --, an item's rank within its
//      wave is the count so far plus the lanes of equal digit below it; the last lane of a digit's group adds the
//      group to the count and clears the entry (the ballots that find such a group without LDS, eight per row, cost
//      four times the vector instructions);
//   2. the 4096 counters are scanned in the order (digit, wave), four per thread;
//   3. the items go to their places.
__device__ inline void two_small_pass(const uint32_t* key_in, const uint16_t* pay_in, uint32_t* key_out, uint16_t* pay_out,
                                      int count, int shift, uint32_t* cnt, uint32_t* part, uint32_t* lanes_a) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  EVX_PASS_TRACE(0);
  const int first = wave * (64 * kTwoSmallPer) + lane;  // a wave's items are consecutive, row by row
  const bool wave_has_items = first - lane < count;      // (wave-uniform)
  unsigned long long* const table = reinterpret_cast<unsigned long long*>(wave < 8 ? lanes_a : key_out) + (wave & 7) * 256;
  // (outside step 2, which lies between barriers, a wave only touches its own counters)
#pragma unroll
  for (int i = 0; i < 4; ++i) cnt[wave * 256 + lane + 64 * i] = 0u;
  uint32_t key[kTwoSmallPer];
  uint16_t pay[kTwoSmallPer];
  int rin[kTwoSmallPer];
#pragma unroll
  for (int r = 0; r < kTwoSmallPer; ++r) {
    key[r] = 0u;
    pay[r] = 0;
    rin[r] = 0;
  }
  if (wave_has_items) {
    const uint4 zero = make_uint4(0u, 0u, 0u, 0u);
    reinterpret_cast<uint4*>(table)[2 * lane] = zero;
    reinterpret_cast<uint4*>(table)[2 * lane + 1] = zero;
    const uint64_t below = (1ull << lane) - 1ull;
#pragma unroll
    for (int r = 0; r < kTwoSmallPer; ++r) {
      const int e = first + r * 64;
      if (e < count) {
        key[r] = key_in[e];
        pay[r] = pay_in[e];
      }
    }
    EVX_PASS_TRACE(1);
#pragma unroll
    for (int r = 0; r < kTwoSmallPer; ++r) {
      const int e = first + r * 64;
      if (e - lane >= count) continue;  // (wave-uniform: a row without items)
      if (e < count) {
        const uint32_t d = (key[r] >> shift) & 255u;
        atomicOr(&table[d], 1ull << lane);
        const uint64_t same = table[d];
        const uint32_t prior = cnt[wave * 256 + d];
        rin[r] = (int)prior + __popcll(same & below);
        if ((same >> lane) == 1ull) {  // the group's last lane
          cnt[wave * 256 + d] = prior + (uint32_t)__popcll(same);
          table[d] = 0ull;
        }
      }
    }
  }
  EVX_PASS_TRACE(2);
  __syncthreads();
  EVX_PASS_TRACE(3);
  // exclusive scan of the counters in the order (digit, wave): thread t has digit t / 4 and the four waves from
  // 4 (t % 4) on (a wave's counters lie together, so that the lanes of a wave meet different banks in steps 1 and 3)
  {
    uint32_t* const mine = cnt + (tid & 3) * 4 * 256 + (tid >> 2);
    const uint32_t c0 = mine[0], c1 = mine[256], c2 = mine[512], c3 = mine[768];
    const uint32_t sum = c0 + c1 + c2 + c3;
    const uint32_t incl = wave_prefix_sum(sum);
    if (lane == 63) part[wave] = incl;
    EVX_PASS_TRACE(4);
    __syncthreads();
    EVX_PASS_TRACE(5);
    uint32_t run = incl - sum + sum_before_wave(part, wave);
    mine[0] = run;
    run += c0;
    mine[256] = run;
    run += c1;
    mine[512] = run;
    run += c2;
    mine[768] = run;
  }
  EVX_PASS_TRACE(6);
  __syncthreads();
  EVX_PASS_TRACE(7);
  if (wave_has_items) {
#pragma unroll
    for (int r = 0; r < kTwoSmallPer; ++r) {
      if (first + r * 64 < count) {
        const uint32_t d = (key[r] >> shift) & 255u;
        const int to = (int)cnt[wave * 256 + d] + rin[r];
        key_out[to] = key[r];
        pay_out[to] = pay[r];
      }
    }
  }
  EVX_PASS_TRACE(8);
  __syncthreads();
  EVX_PASS_TRACE(9);
}

// `passes` passes from the lowest digit up (1 .. 4); returns through the references where the result lies.  vary: the
// bits in which any two keys differ (or more bits); a digit in which no two keys differ needs no pass -- objectives
// that take few values, such as counts or multiples of a step, leave the low bits of their float32 images alike.
__device__ inline void two_small_sort(uint32_t*& key_a, uint16_t*& pay_a, uint32_t*& key_b, uint16_t*& pay_b, int count, int passes,
                                      uint32_t* cnt, uint32_t* part, uint32_t* lanes_a, uint32_t vary = 0xFFFFFFFFu) {
  for (int p = 0; p < passes; ++p) {
    if (((vary >> (8 * p)) & 255u) == 0u) continue;  // (the same in every thread)
    two_small_pass(key_a, pay_a, key_b, pay_b, count, 8 * p, cnt, part, lanes_a);
    uint32_t* tk = key_a;
    key_a = key_b;
    key_b = tk;
    uint16_t* tp = pay_a;
    pay_a = pay_b;
    pay_b = tp;
  }
}

// Grid: one workgroup of kTwoSmallThreads per population; dynamic LDS kTwoSmallLdsBytes.  a.m == 2, a.n <= kTwoSmallRows.
__global__ __launch_bounds__(kTwoSmallThreads) void two_small_kernel(BatchedArgs a) {
  extern __shared__ __attribute__((aligned(16))) uint8_t two_small_lds[];
  __shared__ __attribute__((aligned(16))) uint32_t wave_min[2][16];
  __shared__ __attribute__((aligned(16))) uint32_t part[16];
  __shared__ uint32_t round_count[3];
  __shared__ uint32_t vary_bits[2];  // bits in which the keys of f1 / of f2 differ from those of row 0
  __shared__ __attribute__((aligned(16))) uint32_t wave_first[16];
  uint32_t* key_a = reinterpret_cast<uint32_t*>(two_small_lds);
  uint32_t* key_b = key_a + kTwoSmallRows;
  uint16_t* pay_a = reinterpret_cast<uint16_t*>(key_b + kTwoSmallRows);
  uint16_t* pay_b = pay_a + kTwoSmallRows;
  uint32_t* cnt = reinterpret_cast<uint32_t*>(pay_b + kTwoSmallRows);
  uint32_t* k1 = cnt + kTwoSmallRows;  // ordered keys of the objectives by row
  uint32_t* k2 = k1 + kTwoSmallRows;
  float* dist = reinterpret_cast<float*>(k2 + kTwoSmallRows);  // by position of the output; before that:
  uint32_t* lanes_a = reinterpret_cast<uint32_t*>(dist);       // the lane masks of the sort's first eight waves
  uint16_t* rank16 = reinterpret_cast<uint16_t*>(dist + kTwoSmallRows);  // by row
  uint16_t* lexi = rank16 + kTwoSmallRows;   // row at every position of the (f1, f2, index) order
  uint16_t* perm = lexi + kTwoSmallRows;     // rows by (rank, index)
  uint16_t* order = perm + kTwoSmallRows;    // the selection order

  const int n = a.n;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const float* __restrict__ f = a.f + (int64_t)blockIdx.x * a.f_stride_b;
  auto fitness_at = [&](int i, int k) {
    return f[(int64_t)i * a.f_stride_row + (int64_t)k * a.f_stride_col + (i >= a.n_first ? a.f_second : 0)];
  };

  EVX_BATCH_TRACE(0);
  // ---- keys, and the order of (f1, f2, index).  Where no two rows share their f1 -- the rule for objectives that are
  // computed, not counted -- the rows by (f1, index) are that order: four passes; else the rows by (f2, index) and
  // then, stably, by f1: eight.  Whether two rows share an f1 is asked of a hash table (8192 words in the buffers that
  // the sort does not use yet: open addressing, a row that meets its own key in the table has found a twin).
  bool twin = false;
  {
    uint32_t* const seen = key_b;  // key_b, pay_a, pay_b: 32 KB in a row
    constexpr uint32_t kEmpty = 0xFFFFFFFFu;
    for (int i = tid; i < 2 * kTwoSmallRows / 4; i += kTwoSmallThreads)
      reinterpret_cast<uint4*>(seen)[i] = make_uint4(kEmpty, kEmpty, kEmpty, kEmpty);
    int nan_f1 = 0;
    uint32_t mine1[kTwoSmallPer], mine2[kTwoSmallPer];
    if (tid < 2) vary_bits[tid] = 0u;
#pragma unroll
    for (int r = 0; r < kTwoSmallPer; ++r) {
      const int i = tid + kTwoSmallThreads * r;
      mine1[r] = kEmpty;
      mine2[r] = kEmpty;
      if (i < n) {
        const uint32_t a1 = ordered_key(fitness_at(i, 0)), a2 = ordered_key(fitness_at(i, 1));
        k1[i] = a1;
        k2[i] = a2;
        mine1[r] = a1;
        mine2[r] = a2;
        nan_f1 += a1 == kEmpty ? 1 : 0;  // (the key of a NaN is the table's mark for a free word: counted instead)
      }
    }
    __syncthreads();
    {
      const uint32_t ref1 = k1[0], ref2 = k2[0];
      uint32_t v1 = 0u, v2 = 0u;
#pragma unroll
      for (int r = 0; r < kTwoSmallPer; ++r) {
        if (tid + kTwoSmallThreads * r < n) {
          v1 |= mine1[r] ^ ref1;
          v2 |= mine2[r] ^ ref2;
        }
      }
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) {
        v1 |= (uint32_t)__shfl_xor((int)v1, off);
        v2 |= (uint32_t)__shfl_xor((int)v2, off);
      }
      if (lane == 0) {
        if (v1) atomicOr(&vary_bits[0], v1);
        if (v2) atomicOr(&vary_bits[1], v2);
      }
    }
#pragma unroll
    for (int r = 0; r < kTwoSmallPer; ++r) {
      if (mine1[r] == kEmpty) continue;
      uint32_t at = (mine1[r] * 2654435761u) >> 19;  // 13 bits
      for (int probe = 0; probe < 2 * kTwoSmallRows; ++probe) {
        const uint32_t old = atomicCAS(&seen[at], kEmpty, mine1[r]);
        if (old == kEmpty) break;
        if (old == mine1[r]) {
          twin = true;
          break;
        }
        at = (at + 1u) & (2u * kTwoSmallRows - 1u);
      }
    }
    nan_f1 = wave_sum(nan_f1);
    if (lane == 0) part[wave] = (uint32_t)nan_f1;
    twin = __syncthreads_or(twin) != 0;
    twin |= sum_before_wave(part, 16) > 1u;
  }
  for (int i = tid; i < n; i += kTwoSmallThreads) {
    key_a[i] = twin ? k2[i] : k1[i];
    pay_a[i] = (uint16_t)i;
  }
  __syncthreads();
  EVX_BATCH_TRACE(1);
  two_small_sort(key_a, pay_a, key_b, pay_b, n, 4, cnt, part, lanes_a, vary_bits[twin ? 1 : 0]);
  EVX_BATCH_TRACE(2);
  if (twin) {
    for (int s = tid; s < n; s += kTwoSmallThreads) key_a[s] = k1[pay_a[s]];
    __syncthreads();
    two_small_sort(key_a, pay_a, key_b, pay_b, n, 4, cnt, part, lanes_a, vary_bits[0]);
  }
  for (int s = tid; s < n; s += kTwoSmallThreads) lexi[s] = pay_a[s];
  __syncthreads();
  EVX_BATCH_TRACE(3);

  // ---- the peeling.  A thread holds four consecutive positions of the order.  Out of the sweep: rows with a NaN
  // (nothing compares with them: front 0) and the copies of a row (they take the rank of the first copy, which
  // counts for all of them).  During the peeling the buffers of the sort hold: key_b = copies per first row,
  // pay_b = rank by position.
  uint32_t* copies = key_b;
  uint16_t* rank_at = pay_b;
  uint32_t v[kTwoSmallPer];
  int first_of[kTwoSmallPer];   // position of the first copy (the position itself for a first row)
  bool is_nan[kTwoSmallPer], is_copy[kTwoSmallPer];
  uint32_t last_first = 0u;     // 1 + the last position of this thread that is not a copy, 0 = none
  int nan_rows = 0;
#pragma unroll
  for (int e = 0; e < kTwoSmallPer; ++e) {
    const int s = kTwoSmallPer * tid + e;
    v[e] = kTwoNone;
    is_nan[e] = false;
    is_copy[e] = false;
    first_of[e] = s;
    if (s < n) {
      const int row = lexi[s];
      const uint32_t a1 = k1[row], a2 = k2[row];
      is_nan[e] = a1 == 0xFFFFFFFFu || a2 == 0xFFFFFFFFu;
      if (!is_nan[e] && s > 0) {
        const int before = lexi[s - 1];
        is_copy[e] = k1[before] == a1 && k2[before] == a2;
      }
      if (!is_nan[e] && !is_copy[e]) v[e] = a2;
      if (!is_copy[e]) last_first = (uint32_t)s + 1u;
      nan_rows += is_nan[e] ? 1 : 0;
      copies[s] = 0u;
    }
  }
  {
    // the first copy of a copy: the last position before it that is not one (a prefix maximum)
    const uint32_t incl = ~wave_prefix_min(~last_first);
    const uint32_t excl = ~(uint32_t)__builtin_amdgcn_update_dpp((int)0xFFFFFFFFu, (int)~incl, 0x138, 0xf, 0xf, false);  // wave_shr:1
    if (lane == 63) wave_first[wave] = incl;
    if (tid < 3) round_count[tid] = 0u;
    __syncthreads();
    uint32_t carry = max(excl, max_before_wave(wave_first, wave));
#pragma unroll
    for (int e = 0; e < kTwoSmallPer; ++e) {
      const int s = kTwoSmallPer * tid + e;
      if (s < n) {
        if (!is_copy[e]) carry = (uint32_t)s + 1u;
        first_of[e] = (int)carry - 1;  // (a copy always has a first row before it)
        if (is_copy[e]) atomicAdd(&copies[first_of[e]], 1u);
      }
    }
    nan_rows = (int)wave_sum(nan_rows);
    if (lane == 0 && nan_rows != 0) atomicAdd(&round_count[0], (uint32_t)nan_rows);
  }
  const int stop = a.stop_count;
  EVX_BATCH_TRACE(4);
  int group[kTwoSmallPer];       // a first row and its copies
  uint16_t ranked[kTwoSmallPer];  // (in registers: a round must not wait for LDS more often than it has to)
#pragma unroll
  for (int e = 0; e < kTwoSmallPer; ++e) {
    group[e] = 1;
    ranked[e] = is_nan[e] ? (uint16_t)0 : kTwoSmallUnset;
  }
  int total = 0, worst = 0, nv = 0;
  // A wave all of whose rows are ranked (or that never had any) only keeps the barriers and the count of the rounds
  // company: sixteen waves share the compute unit's four vector units, and what one of them does not issue the others
  // issue sooner.
  bool wave_live = true;     // (wave-uniform)
  bool wave_copies = false;  // some first row of this wave has copies: the rows of a round are then added, not counted
  for (int round = 0;; ++round) {
    uint32_t running = kTwoNone;
    if (wave_live) {
      uint32_t tmin = kTwoNone;
#pragma unroll
      for (int e = 0; e < kTwoSmallPer; ++e) tmin = min(tmin, v[e]);
      const uint32_t incl = wave_prefix_min(tmin);
      running = (uint32_t)__builtin_amdgcn_update_dpp((int)kTwoNone, (int)incl, 0x138, 0xf, 0xf, false);  // wave_shr:1
      if (lane == 63) wave_min[round & 1][wave] = incl;
    } else if (lane == 63) {
      wave_min[round & 1][wave] = kTwoNone;  // (not earlier: the round before may still be reading the other word)
    }
    if (round == 2) EVX_PASS_TRACE(11);
    __syncthreads();  // (the first one also completes the copies' counts)
    if (round == 2) EVX_PASS_TRACE(12);
    if (round == 0) {
      bool any = false;
#pragma unroll
      for (int e = 0; e < kTwoSmallPer; ++e)
        if (kTwoSmallPer * tid + e < n) {
          group[e] = 1 + (int)copies[kTwoSmallPer * tid + e];
          any |= group[e] > 1;
        }
      wave_copies = __builtin_amdgcn_ballot_w64(any) != 0ull;
    }
    // (the counter of the next round: last read after the barrier before this one)
    if (tid == 0) round_count[(round + 1) % 3] = 0u;
    if (round > 0) {
      const int size = (int)round_count[(round - 1) % 3];
      total += size;
      if (size == 0 || total >= stop) {
        worst = round - 1;
        nv = size;
        break;
      }
    }
    if (!wave_live) continue;
    running = min(running, min_before_wave(wave_min[round & 1], wave));
    if (round == 2) EVX_PASS_TRACE(13);
    int add = 0;
    bool left = false;
    bool now[kTwoSmallPer];
#pragma unroll
    for (int e = 0; e < kTwoSmallPer; ++e) {
      const uint32_t mine = v[e];
      now[e] = mine < running;  // (a row out of the sweep holds kTwoNone, which is below nothing)
      running = min(running, mine);
      if (now[e]) {
        ranked[e] = (uint16_t)round;
        v[e] = kTwoNone;
      }
      left |= v[e] != kTwoNone;
    }
    if (round == 2) EVX_PASS_TRACE(14);
    if (wave_copies) {
#pragma unroll
      for (int e = 0; e < kTwoSmallPer; ++e) add += now[e] ? group[e] : 0;
      add = wave_sum(add);
    } else {
#pragma unroll
      for (int e = 0; e < kTwoSmallPer; ++e) add += __popcll(__builtin_amdgcn_ballot_w64(now[e]));
    }
    if (lane == 0 && add != 0) atomicAdd(&round_count[round % 3], (uint32_t)add);
    wave_live = __builtin_amdgcn_ballot_w64(left) != 0ull;
    if (round == 2) EVX_PASS_TRACE(15);
  }
  const int worst_start = total - nv;
  EVX_BATCH_TRACE(5);
#pragma unroll
  for (int e = 0; e < kTwoSmallPer; ++e)
    if (kTwoSmallPer * tid + e < n) rank_at[kTwoSmallPer * tid + e] = ranked[e];
  __syncthreads();
  // ranks by row: the copies take that of their first row
#pragma unroll
  for (int e = 0; e < kTwoSmallPer; ++e) {
    const int s = kTwoSmallPer * tid + e;
    if (s < n) rank16[lexi[s]] = rank_at[first_of[e]];
  }
  __syncthreads();
  if (a.rank_all)
    for (int i = tid; i < n; i += kTwoSmallThreads)
      a.rank_all[(int64_t)blockIdx.x * n + i] = rank16[i] == kTwoSmallUnset ? kRankUnset : (int)rank16[i];
  if (a.out_f == nullptr) return;  // rank-only mode

  EVX_BATCH_TRACE(6);
  // ---- the rows by (rank, index): the rows are in index order, the sort is stable (the rows not ranked come last)
  key_a = reinterpret_cast<uint32_t*>(two_small_lds);
  key_b = key_a + kTwoSmallRows;
  pay_a = reinterpret_cast<uint16_t*>(key_b + kTwoSmallRows);
  pay_b = pay_a + kTwoSmallRows;
  for (int i = tid; i < n; i += kTwoSmallThreads) {
    key_a[i] = rank16[i];
    pay_a[i] = (uint16_t)i;
  }
  __syncthreads();
  two_small_sort(key_a, pay_a, key_b, pay_b, n, worst < 255 ? 1 : 2, cnt, part, lanes_a);
  for (int p = tid; p < n; p += kTwoSmallThreads) perm[p] = pay_a[p];
  __syncthreads();

  // ---- crowding distances of the last front (candidate q = perm[worst_start + q], in index order) and the order
  // by (distance descending, index): non_dominate.py:209-231 with the mask rank == worst, :253
  const int need = stop - worst_start;
  EVX_BATCH_TRACE(7);
  auto better_fronts = [&]() {  // (the distances share their LDS with the sort: only once the last sort is over)
    for (int p = tid; p < stop; p += kTwoSmallThreads) {
      dist[p] = -INFINITY;
      if (p < worst_start) order[p] = perm[p];
    }
    __syncthreads();
  };
  if (nv <= kTwoSmallCounting) {
    better_fronts();
    // by counting: thread q is candidate q; tile and below lie in the sort's buffers
    uint64_t* tile = reinterpret_cast<uint64_t*>(two_small_lds);                   // nv + 4 entries
    float* scost = reinterpret_cast<float*>(tile + (kTwoSmallCounting + 4));       // by position
    int* below = reinterpret_cast<int*>(scost + kTwoSmallCounting);
    const bool cand = tid < nv;
    const int row = cand ? perm[worst_start + tid] : 0;
    bool boundary = false;
    float acc = 0.0f;
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      const uint32_t ck = cand ? (k == 0 ? k1[row] : k2[row]) : 0u;
      __syncthreads();
      if (tid < nv + 4) tile[tid] = cand ? ((uint64_t)ck << 32) | (uint32_t)tid : ~0ull;
      if (tid < 4 && nv + tid >= kTwoSmallThreads) tile[nv + tid] = ~0ull;
      const int p = position_by_counting(tile, below, nv, tid, kTwoSmallThreads);
      if (cand) scost[p] = cost_of_key(ck);
      __syncthreads();
      if (cand) {
        if (p == 0 || p == nv - 1) {
          boundary = true;
        } else {
          const float term = (scost[p + 1] - scost[p - 1]) / (scost[nv - 1] - scost[0]);
          acc = k == 0 ? term : acc + term;
        }
      }
    }
    const float d = boundary ? INFINITY : acc;
    __syncthreads();
    if (tid < nv + 4) tile[tid] = cand ? ((uint64_t)ordered_key(-d) << 32) | (uint32_t)tid : ~0ull;
    if (tid < 4 && nv + tid >= kTwoSmallThreads) tile[nv + tid] = ~0ull;
    const int p = position_by_counting(tile, below, nv, tid, kTwoSmallThreads);
    if (cand && p < need) {
      order[worst_start + p] = (uint16_t)row;
      dist[worst_start + p] = d;
    }
  } else {
    // by the radix sort: a thread has candidates q = tid + 1024 r; scost (by position) and pos (by candidate) lie
    // in the counters' neighbours k-independent: scost in `dist`'s tail is not free, so they take the copy buffers
    float acc[kTwoSmallPer];
    bool boundary[kTwoSmallPer];
#pragma unroll
    for (int r = 0; r < kTwoSmallPer; ++r) {
      acc[r] = 0.0f;
      boundary[r] = false;
    }
    for (int k = 0; k < 2; ++k) {
      key_a = reinterpret_cast<uint32_t*>(two_small_lds);
      key_b = key_a + kTwoSmallRows;
      pay_a = reinterpret_cast<uint16_t*>(key_b + kTwoSmallRows);
      pay_b = pay_a + kTwoSmallRows;
      for (int q = tid; q < nv; q += kTwoSmallThreads) {
        const int row = perm[worst_start + q];
        key_a[q] = k == 0 ? k1[row] : k2[row];
        pay_a[q] = (uint16_t)q;
      }
      __syncthreads();
      two_small_sort(key_a, pay_a, key_b, pay_b, nv, 4, cnt, part, lanes_a);  // four passes: the result is where it started
      // position of every candidate: into the other payload buffer
      for (int p = tid; p < nv; p += kTwoSmallThreads) pay_b[pay_a[p]] = (uint16_t)p;
      __syncthreads();
      const float span = cost_of_key(key_a[nv - 1]) - cost_of_key(key_a[0]);
#pragma unroll
      for (int r = 0; r < kTwoSmallPer; ++r) {
        const int q = tid + kTwoSmallThreads * r;
        if (q < nv) {
          const int p = pay_b[q];
          if (p == 0 || p == nv - 1) {
            boundary[r] = true;
          } else {
            const float term = (cost_of_key(key_a[p + 1]) - cost_of_key(key_a[p - 1])) / span;
            acc[r] = k == 0 ? term : acc[r] + term;
          }
        }
      }
      __syncthreads();
    }
    key_a = reinterpret_cast<uint32_t*>(two_small_lds);
    key_b = key_a + kTwoSmallRows;
    pay_a = reinterpret_cast<uint16_t*>(key_b + kTwoSmallRows);
    pay_b = pay_a + kTwoSmallRows;
    float* d_of = reinterpret_cast<float*>(cnt + kTwoSmallRows);  // (= k1: no longer needed once the keys below are built)
    float d_mine[kTwoSmallPer];
#pragma unroll
    for (int r = 0; r < kTwoSmallPer; ++r) d_mine[r] = boundary[r] ? INFINITY : acc[r];
    __syncthreads();
#pragma unroll
    for (int r = 0; r < kTwoSmallPer; ++r) {
      const int q = tid + kTwoSmallThreads * r;
      if (q < nv) {
        key_a[q] = ordered_key(-d_mine[r]);
        pay_a[q] = (uint16_t)q;
        d_of[q] = d_mine[r];
      }
    }
    __syncthreads();
    two_small_sort(key_a, pay_a, key_b, pay_b, nv, 4, cnt, part, lanes_a);
    better_fronts();
    for (int p = tid; p < need; p += kTwoSmallThreads) {
      const int q = pay_a[p];
      order[worst_start + p] = perm[worst_start + q];
      dist[worst_start + p] = d_of[q];
    }
  }
  __syncthreads();
  EVX_BATCH_TRACE(8);

  // ---- the selected rows
  const int topk = stop;
  const int64_t ob = (int64_t)blockIdx.x * topk;
  for (int p = tid; p < topk; p += kTwoSmallThreads) {
    const int src = order[p];
    a.out_rank[ob + p] = (int)rank16[src];
    a.out_dist[ob + p] = dist[p];
    a.out_f[(ob + p) * 2] = fitness_at(src, 0);
    a.out_f[(ob + p) * 2 + 1] = fitness_at(src, 1);
  }
  if (a.x != nullptr) {
    const uint8_t* __restrict__ xb = a.x + (int64_t)blockIdx.x * a.x_stride_b;
    uint8_t* __restrict__ dst = a.out_x + ob * a.x_row_bytes;
    const int64_t row_units = a.x_row_bytes / a.x_unit;
    const int64_t units = row_units * topk;
    if (a.x_unit >= 4 && units < (1ll << 31)) {
      if (a.x_unit == 16)
        gather_units<uint4>(xb, dst, order, a.x_row_stride, (uint32_t)row_units, (uint32_t)units, tid, kTwoSmallThreads, a.n_first,
                            a.x_second);
      else
        gather_units<uint32_t>(xb, dst, order, a.x_row_stride, (uint32_t)row_units, (uint32_t)units, tid, kTwoSmallThreads,
                               a.n_first, a.x_second);
    } else {
      for (int p = wave; p < topk; p += kTwoSmallThreads / 64) {
        const int src = order[p];
        const uint8_t* __restrict__ sp = xb + (int64_t)src * a.x_row_stride + (src >= a.n_first ? a.x_second : 0);
        uint8_t* __restrict__ dp = dst + (int64_t)p * a.x_row_bytes;
        if (a.x_unit == 4) {
          for (int64_t b = lane * 4; b < a.x_row_bytes; b += 64 * 4)
            *reinterpret_cast<uint32_t*>(dp + b) = *reinterpret_cast<const uint32_t*>(sp + b);
        } else {
          for (int64_t b = lane; b < a.x_row_bytes; b += 64) dp[b] = sp[b];
        }
      }
    }
  }
  EVX_BATCH_TRACE(9);
}

}  // namespace evx
