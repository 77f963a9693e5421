// The slot sort of a mid-sized population (4097 .. 32768 rows) in ONE launch, with no dependence between workgroups.
//
// What it produces is what prepare_kernel and the four kernels of the bucket sort (order.hpp) produce together: the
// fitness as a structure of arrays in original order, the rows relabelled by ascending (row key, original index) --
// slot-ordered fitness, keys, first slot of every key, slot <-> original index -- the flag that tells whether a value
// is NaN or infinite, and the cleared state region.  Five launches of a few microseconds each are what the smallest
// kernel costs on this device five times over; here every workgroup does all the O(n) work for itself and the O(n)
// work is kept to two passes over the rows:
//   1. 256 rows at pseudo-random positions are the sample: ranked by counting, they cut the (key, index) order into as
//      many ranges as there are workgroups -- whatever the distribution of the keys, and because the index is part of
//      what is cut, even thousands of equal rows are dealt out evenly;
//   2. one pass over the rows (a thread takes row t, t + 1024, ...): the key of the row is computed, the rows before
//      the workgroup's range are counted (its first slot) and the rows inside it collected in LDS;
//   3. every member is placed by counting the members before it.
// A range that holds more members than the LDS list (no sample fell into a fifth of the population: not something a
// population does, but nothing rules it out) is placed by counting over all rows instead: slow and still exact.
#pragma once

#include "common.hpp"
#include "dominance.hpp"
#include "order.hpp"
#include "peel.hpp"

namespace evx {

constexpr int kOneSortThreads = 1024;
constexpr int kOneSortSamples = 256;
constexpr int kOneSortCap = 4096;        // members of a range held in LDS
constexpr int kOneSortMinRows = 4097;    // (smaller populations: small_sort_kernel)
constexpr int kOneSortMaxRows = 32768;
constexpr int64_t kOneSortMaxValues = 131072;  // n * m: every workgroup reads every value

__device__ inline bool pair_less(double ka, int ia, double kb, int ib) { return ka < kb || (ka == kb && ia < ib); }

__global__ __launch_bounds__(kOneSortThreads) void one_sort_kernel(
    const float* __restrict__ f, int64_t stride_row, int64_t stride_col, int n_first, const float* __restrict__ f2,
    int64_t stride_row2, int64_t stride_col2, int n, int m, int npad, float* __restrict__ xs, double* __restrict__ key_scratch,
    SortParam* __restrict__ param_out, uint64_t* __restrict__ key_sorted, uint32_t* __restrict__ kid_sorted,
    float* __restrict__ xs_sorted, int* __restrict__ orig_of, int* __restrict__ slot_of, uint32_t* __restrict__ zero_words,
    int64_t n_zero_words, int cap) {
  __shared__ double s_key[kOneSortSamples];
  __shared__ int s_idx[kOneSortSamples];
  __shared__ int s_rank[kOneSortSamples];
  __shared__ double cut_key[kOneSortSamples];
  __shared__ int cut_idx[kOneSortSamples];
  __shared__ double mem_key[kOneSortCap];
  __shared__ int mem_idx[kOneSortCap];
  __shared__ int counters[4];
  __shared__ int red[2][kOneSortThreads / 64];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  auto value = [&](int i, int k) {
    return i < n_first ? f[(int64_t)i * stride_row + k * stride_col] : f2[(int64_t)(i - n_first) * stride_row2 + k * stride_col2];
  };
  auto row_key = [&](int i) {
    uint64_t s = 0;
    for (int k = 0; k < m; ++k) s += (uint64_t)key_weight(k) * ordered_key(value(i, k));
    return (double)s;  // below 2^53: exact
  };
  // ---- 1. the sample and its order
  if (tid < kOneSortSamples) {
    const int span = n / kOneSortSamples > 0 ? n / kOneSortSamples : 1;
    int p = (int)(((int64_t)tid * n) / kOneSortSamples) + (int)((((uint32_t)tid * 2654435761u) >> 8) % (uint32_t)span);
    if (p >= n) p = n - 1;
    s_key[tid] = row_key(p);
    s_idx[tid] = p;
    s_rank[tid] = 0;
  }
  if (tid < 4) counters[tid] = 0;
  __syncthreads();
  {
    // sample s against a quarter of the samples (the quarter is the same in all lanes of a wave: broadcast reads);
    // a row sampled twice is told apart by its place in the sample
    const int s = tid & (kOneSortSamples - 1), part = tid / kOneSortSamples;
    const double ks = s_key[s];
    const int is = s_idx[s];
    int smaller = 0;
    constexpr int kPer = kOneSortSamples / (kOneSortThreads / kOneSortSamples);
    for (int q = part * kPer; q < part * kPer + kPer; ++q) {
      const double kq = s_key[q];
      const int iq = s_idx[q];
      smaller += kq < ks || (kq == ks && (iq < is || (iq == is && q < s)));
    }
    atomicAdd(&s_rank[s], smaller);
  }
  __syncthreads();
  if (tid < kOneSortSamples) {
    cut_key[s_rank[tid]] = s_key[tid];
    cut_idx[s_rank[tid]] = s_idx[tid];
  }
  __syncthreads();
  // the range of this workgroup: [lo, hi) in (key, index) order; gridDim.x is a power of two up to kOneSortSamples
  const int b = blockIdx.x, step = kOneSortSamples / (int)gridDim.x;
  const bool first = b == 0, last = b == (int)gridDim.x - 1;
  const double lo_key = first ? -1.0 : cut_key[b * step], hi_key = last ? (double)INFINITY : cut_key[last ? 0 : (b + 1) * step];
  const int lo_idx = first ? -1 : cut_idx[b * step], hi_idx = last ? 0x7FFFFFFF : cut_idx[last ? 0 : (b + 1) * step];
  // ---- 2. one pass over the rows (row t, t + 1024, ... are this thread's): the rows before the range are counted,
  // the rows inside it collected.  Eight rows at a time, the loads of one objective for all eight in flight together.
  int before_range = 0, keys_before = 0;  // rows below lo; rows whose key is below lo's key
  uint32_t member_rows = 0;               // bit r: this thread's r-th row is a member (n <= 32 * 1024)
  bool bad = false;
  constexpr int kUnroll = 8;
  const int rows_per_thread = (n + kOneSortThreads - 1) / kOneSortThreads;
  for (int r0 = 0; r0 < rows_per_thread; r0 += kUnroll) {
    uint64_t sum[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) sum[u] = 0;
    for (int k = 0; k < m; ++k) {
      float v[kUnroll];
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        const int i = tid + (r0 + u) * kOneSortThreads;
        v[u] = i < n ? value(i, k) : 0.0f;
      }
      const uint64_t weight = key_weight(k);
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        sum[u] += weight * ordered_key(v[u]);
        bad |= !(fabsf(v[u]) <= 3.4028234663852886e38f);  // NaN or infinite (the stand-in of a missing row is 0)
      }
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const int i = tid + (r0 + u) * kOneSortThreads;
      if (i < n) {
        const double key = (double)sum[u];  // below 2^53: exact
        const bool below = pair_less(key, i, lo_key, lo_idx);
        before_range += below;
        keys_before += key < lo_key;
        if (!below && pair_less(key, i, hi_key, hi_idx)) {
          member_rows |= 1u << (r0 + u);
          const int e = atomicAdd(&counters[0], 1);
          if (e < cap) {
            mem_key[e] = key;
            mem_idx[e] = i;
          }
        }
      }
    }
  }
  before_range = wave_sum(before_range);
  keys_before = wave_sum(keys_before);
  if (lane == 0) {
    red[0][wave] = before_range;
    red[1][wave] = keys_before;
  }
  const int any_bad = __syncthreads_or(bad);
  before_range = 0;
  keys_before = 0;
#pragma unroll
  for (int v = 0; v < kOneSortThreads / 64; ++v) {
    before_range += red[0][v];
    keys_before += red[1][v];
  }
  const int members = counters[0];
  auto place = [&](int i, double ki, int slot, int kid, int sub, int lanes) {
    // the outputs of one row, shared by `lanes` lanes (sub = this lane's number among them)
    if (sub == 0) {
      orig_of[slot] = i;
      slot_of[i] = slot;
      key_sorted[slot] = (uint64_t)ki;
      kid_sorted[slot] = (uint32_t)kid;  // first slot holding this key: equal ids <=> equal keys
    }
    // -0.0 is stored as +0.0: every comparison reads the same, and differences of equal values are +0.0
    for (int k = sub; k < m; k += lanes) xs_sorted[(int64_t)k * npad + slot] = value(i, k) + 0.0f;
  };
  if (members <= cap) {
    // sixteen lanes per member count the members before it (and those of smaller key)
    const int sub = tid & 15;
    for (int e = tid >> 4; e < members; e += kOneSortThreads / 16) {
      const double ke = mem_key[e];
      const int ie = mem_idx[e];
      int before = 0, smaller = 0;
      for (int q = sub; q < members; q += 16) {
        const double kq = mem_key[q];
        smaller += kq < ke;
        before += kq < ke || (kq == ke && mem_idx[q] < ie);
      }
      before = group16_sum(before);
      smaller = group16_sum(smaller);
      // rows before the range have keys up to lo's key: all of them are smaller than a larger key, and of a member
      // that shares lo's key those whose key is below it
      place(ie, ke, before_range + before, (ke > lo_key ? before_range : keys_before) + smaller, sub, 16);
    }
  } else {
    // more members than the list holds: every member is placed by counting over all rows (the keys go through
    // memory: every workgroup that gets here writes the same values)
    for (int i = tid; i < n; i += kOneSortThreads) key_scratch[i] = row_key(i);
    __syncthreads();
    for (int r = 0; r < rows_per_thread; ++r) {
      if ((member_rows >> r) & 1u) {
        const int i = tid + r * kOneSortThreads;
        const double key = row_key(i);
        int before = 0, smaller = 0;
        for (int q = 0; q < n; ++q) {
          const double kq = key_scratch[q];
          smaller += kq < key;
          before += kq < key || (kq == key && q < i);
        }
        place(i, key, before, smaller, 0, 1);
      }
    }
  }
  // ---- the fitness in original order and the padding behind the n-th row and slot, a share per workgroup
  {
    const int per = (npad + (int)gridDim.x - 1) / (int)gridDim.x;
    const int end = min(npad, (b + 1) * per);
    for (int i = b * per + tid; i < end; i += kOneSortThreads) {
      if (i < n) {
        for (int k = 0; k < m; ++k) xs[(int64_t)k * npad + i] = value(i, k);
      } else {
        orig_of[i] = -1;
        key_sorted[i] = ~0ull;
        kid_sorted[i] = (uint32_t)i;
        for (int k = 0; k < m; ++k) {
          xs[(int64_t)k * npad + i] = __uint_as_float(0x7FC00000u);
          xs_sorted[(int64_t)k * npad + i] = __uint_as_float(0x7FC00000u);
        }
      }
    }
  }
  if (b == 0 && tid == 0) {
    SortParam sp;
    sp.kmin = 0ull;
    sp.shift = 0;
    sp.buckets = 0;
    sp.nonfinite = any_bad != 0;
    sp.totals_valid = 0;
    sp.orders_valid = 0;
    *param_out = sp;
  }
  const int64_t gtid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  for (int64_t w = gtid; w < n_zero_words; w += (int64_t)gridDim.x * blockDim.x) zero_words[w] = 0u;
}

}  // namespace evx
