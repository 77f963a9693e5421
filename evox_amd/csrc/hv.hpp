// Monte-Carlo hypervolume: the other users of a pairwise "no worse in every objective" test, points
// against samples instead of rows against rows.
//
// HypE's contributions (src/evox/algorithms/mo/hype.py:12-39):
//   pds[s, i] = all_k fit[i, k] - sample[s, k] <= 0                               (hype.py:30)
//   ds[s]     = number of points with pds[s, .], minus one when it is not zero    (hype.py:31-32)
//   f[i]      = sum_s pds[s, i] ? alpha[ds[s]] : 0                                (hype.py:34-36)
// The metric (src/evox/metrics/hv.py:13-19):
//   covered[s] = any_i all_k sample[s, k] < point[i, k]                           (hv.py:18)
//
// One side of a pair sits in the lanes, the other side streams past as scalar operands, eight at a time
// (consecutive coordinates of the transposed arrays, so one scalar load brings eight of them).  Both
// sides of every kernel are cut into chunks (grid x = lane side, grid y = streamed side) so that a few
// thousand points against ten thousand samples still fill the device.
#pragma once

#include "common.hpp"

namespace evx {

constexpr int kHvChunk = 256;        // samples per partial sum of the contributions, at least
constexpr int kHvPointChunk = 128;   // points per partial cover count of the contributions, at least
constexpr int kHvMaxChunks = 64;     // chunks of either kind, at most (bounds the workspace)
constexpr int kHvCoverChunk = 1024;  // points per block of the metric
constexpr int kHvRegs = 16;          // objectives held in registers; more are re-read from memory

// Length of the chunks that cut `count` items into at most kHvMaxChunks pieces of at least `least` items
// (a multiple of eight, the streaming unit).
__host__ __device__ inline int hv_chunk_length(int64_t count, int least) {
  int64_t len = (count + kHvMaxChunks - 1) / kHvMaxChunks;
  if (len < least) len = least;
  return (int)((len + 7) & ~7ll);
}

// The reference's test is on the difference (hype.py:30): inf - inf is NaN and fails it.
__device__ inline bool hv_no_worse(float fit, float sample) { return fit - sample <= 0.0f; }

// cover[c][s] = number of points i of chunk c with pds[s, i]; lane = sample, the chunk's points stream past.
// fit_t is (m, n) and samples_t is (m, n_sample), both row-major.  grid = (sample blocks, point chunks).
__global__ __launch_bounds__(256) void hv_cover_count_kernel(const float* __restrict__ fit_t, const float* __restrict__ samples_t,
                                                             int n, int m, int n_sample, int chunk,
                                                             int32_t* __restrict__ cover) {
  const int s = blockIdx.x * blockDim.x + threadIdx.x;
  const int sc = s < n_sample ? s : n_sample - 1;
  const int i0 = blockIdx.y * chunk;
  const int i1 = min(n, i0 + chunk);
  int count = 0;
  if (m <= kHvRegs) {
    float sv[kHvRegs];
#pragma unroll
    for (int k = 0; k < kHvRegs; ++k) sv[k] = k < m ? samples_t[(int64_t)k * n_sample + sc] : 0.0f;
    int i = i0;
    for (; i + 8 <= i1; i += 8) {
      bool c[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) c[u] = true;
#pragma unroll
      for (int k = 0; k < kHvRegs; ++k) {
        if (k < m) {
          const float* __restrict__ row = fit_t + (int64_t)k * n + i;
#pragma unroll
          for (int u = 0; u < 8; ++u) c[u] &= hv_no_worse(row[u], sv[k]);
        }
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) count += c[u] ? 1 : 0;
    }
    for (; i < i1; ++i) {
      bool c = true;
#pragma unroll
      for (int k = 0; k < kHvRegs; ++k)
        if (k < m) c &= hv_no_worse(fit_t[(int64_t)k * n + i], sv[k]);
      count += c ? 1 : 0;
    }
  } else {
    for (int i = i0; i < i1; ++i) {
      bool c = true;
      for (int k = 0; k < m; ++k) c &= hv_no_worse(fit_t[(int64_t)k * n + i], samples_t[(int64_t)k * n_sample + sc]);
      count += c ? 1 : 0;
    }
  }
  if (s < n_sample) cover[(int64_t)blockIdx.y * n_sample + s] = count;
}

// weight[s] = alpha[max(ds[s], 0)], ds[s] = (sum of the chunk counts of sample s) - 1.
__global__ __launch_bounds__(256) void hv_sample_weight_kernel(const int32_t* __restrict__ cover, const float* __restrict__ alpha,
                                                               int point_chunks, int n_sample, float* __restrict__ weight) {
  const int s = blockIdx.x * blockDim.x + threadIdx.x;
  if (s >= n_sample) return;
  int covered = 0;
  for (int c = 0; c < point_chunks; ++c) covered += cover[(int64_t)c * n_sample + s];
  weight[s] = alpha[covered == 0 ? 0 : covered - 1];
}

// partial[chunk][i] = sum over the samples s of the chunk, in ascending s, of (pds[s, i] ? weight[s] : 0);
// lane = point, the chunk's samples stream past.  grid = (point blocks, sample chunks).
__global__ __launch_bounds__(256) void hv_point_partial_kernel(const float* __restrict__ fit_t, const float* __restrict__ samples_t,
                                                               const float* __restrict__ weight, int n, int m, int n_sample,
                                                               int chunk, float* __restrict__ partial) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  const int ic = i < n ? i : n - 1;
  const int s0 = blockIdx.y * chunk;
  const int s1 = min(n_sample, s0 + chunk);
  float acc = 0.0f;
  if (m <= kHvRegs) {
    float fv[kHvRegs];
#pragma unroll
    for (int k = 0; k < kHvRegs; ++k) fv[k] = k < m ? fit_t[(int64_t)k * n + ic] : 0.0f;
    int s = s0;
    for (; s + 8 <= s1; s += 8) {
      bool c[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) c[u] = true;
#pragma unroll
      for (int k = 0; k < kHvRegs; ++k) {
        if (k < m) {
          const float* __restrict__ row = samples_t + (int64_t)k * n_sample + s;
#pragma unroll
          for (int u = 0; u < 8; ++u) c[u] &= hv_no_worse(fv[k], row[u]);
        }
      }
      const float* __restrict__ w = weight + s;
#pragma unroll
      for (int u = 0; u < 8; ++u) acc += c[u] ? w[u] : 0.0f;
    }
    for (; s < s1; ++s) {
      bool c = true;
#pragma unroll
      for (int k = 0; k < kHvRegs; ++k)
        if (k < m) c &= hv_no_worse(fv[k], samples_t[(int64_t)k * n_sample + s]);
      acc += c ? weight[s] : 0.0f;
    }
  } else {
    for (int s = s0; s < s1; ++s) {
      bool c = true;
      for (int k = 0; k < m; ++k) c &= hv_no_worse(fit_t[(int64_t)k * n + ic], samples_t[(int64_t)k * n_sample + s]);
      acc += c ? weight[s] : 0.0f;
    }
  }
  if (i < n) partial[(int64_t)blockIdx.y * n + i] = acc;
}

// out[i] = (sum of the partial sums of point i, in chunk order) * scale.
__global__ __launch_bounds__(256) void hv_point_total_kernel(const float* __restrict__ partial, int n, int chunks, float scale,
                                                             float* __restrict__ out) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  float acc = 0.0f;
  for (int c = 0; c < chunks; ++c) acc += partial[(int64_t)c * n + i];
  out[i] = acc * scale;
}

// ---------------------------------------------------------------- the metric

// flag[s] becomes 1 when some point of the block's chunk exceeds sample s strictly in every objective (a NaN
// on either side compares false).  Lane = sample, points stream past; a wave stops as soon as all of its
// samples are covered, and skips the chunk when an earlier block has covered them already (flags only go
// from 0 to 1, so reading an old 0 costs work, not correctness).  flag must be zero at the start.
// points_t is (m, n), samples_t is (m, n_sample), row-major.  grid = (sample blocks, point chunks).
__global__ __launch_bounds__(256) void hv_covered_kernel(const float* __restrict__ points_t, const float* __restrict__ samples_t,
                                                         int n, int m, int n_sample, uint32_t* __restrict__ flag) {
  const int s = blockIdx.x * blockDim.x + threadIdx.x;
  const bool live = s < n_sample;
  const int sc = live ? s : n_sample - 1;
  const int i0 = blockIdx.y * kHvCoverChunk;
  const int i1 = min(n, i0 + kHvCoverChunk);
  const bool before = live ? __builtin_nontemporal_load(flag + sc) != 0u : true;
  bool cov = before;
  if (__builtin_amdgcn_ballot_w64(!cov) == 0ull) return;
  if (m <= kHvRegs) {
    float sv[kHvRegs];
#pragma unroll
    for (int k = 0; k < kHvRegs; ++k) sv[k] = k < m ? samples_t[(int64_t)k * n_sample + sc] : 0.0f;
    int i = i0;
    for (; i + 8 <= i1; i += 8) {
      bool c[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) c[u] = true;
#pragma unroll
      for (int k = 0; k < kHvRegs; ++k) {
        if (k < m) {
          const float* __restrict__ row = points_t + (int64_t)k * n + i;
#pragma unroll
          for (int u = 0; u < 8; ++u) c[u] &= sv[k] < row[u];
        }
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) cov |= c[u];
      if (__builtin_amdgcn_ballot_w64(!cov) == 0ull) break;
    }
    if (__builtin_amdgcn_ballot_w64(!cov) != 0ull) {
      for (i = max(i, i0); i < i1; ++i) {  // the tail of the chunk (fewer than eight points)
        bool c = true;
#pragma unroll
        for (int k = 0; k < kHvRegs; ++k)
          if (k < m) c &= sv[k] < points_t[(int64_t)k * n + i];
        cov |= c;
      }
    }
  } else {
    for (int i = i0; i < i1 && __builtin_amdgcn_ballot_w64(!cov) != 0ull; ++i) {
      bool c = true;
      for (int k = 0; k < m; ++k) c &= samples_t[(int64_t)k * n_sample + sc] < points_t[(int64_t)k * n + i];
      cov |= c;
    }
  }
  if (live && cov && !before) flag[s] = 1u;
}

// out[0] += number of set flags (out must be zero at the start; integer adds, so any order gives the count).
__global__ __launch_bounds__(256) void hv_covered_total_kernel(const uint32_t* __restrict__ flag, int n_sample,
                                                               unsigned long long* __restrict__ out) {
  __shared__ int part[4];
  int acc = 0;
  for (int s = blockIdx.x * blockDim.x + threadIdx.x; s < n_sample; s += gridDim.x * blockDim.x) acc += flag[s] != 0u ? 1 : 0;
  for (int d = 32; d > 0; d >>= 1) acc += __shfl_xor(acc, d);
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = acc;
  __syncthreads();
  if (threadIdx.x == 0) {
    const int total = part[0] + part[1] + part[2] + part[3];
    if (total != 0) atomicAdd(out, (unsigned long long)total);
  }
}

}  // namespace evx
