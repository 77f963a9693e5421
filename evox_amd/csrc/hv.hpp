// Monte-Carlo hypervolume contributions of HypE (src/evox/algorithms/mo/hype.py:12-39): the other user of
// the pairwise "no worse in every objective" test.  Points against samples instead of rows against rows:
//   pds[s, i] = all_k fit[i, k] <= sample[s, k]                                  (hype.py:30)
//   ds[s]     = number of points with pds[s, .], minus one when it is not zero    (hype.py:31-32)
//   f[i]      = sum_s pds[s, i] ? alpha[ds[s]] : 0                                (hype.py:34-36)
// Same compare scheme as the dominance kernel: one side of the pair sits in the lanes, the other side
// streams past as scalar operands, so a `<=` is one v_cmp with an SGPR operand and the per-objective
// masks are combined on the scalar unit.
#pragma once

#include "common.hpp"

namespace evx {

constexpr int kHvChunk = 1024;  // samples per partial sum

// weight[s] = alpha[max(ds[s], 0)] for sample s (ds as above); lane = sample, points stream past.
// fit_t is (m, n) and samples_t is (m, n_sample), both row-major.
__global__ __launch_bounds__(256) void hv_sample_weight_kernel(const float* __restrict__ fit_t, const float* __restrict__ samples_t,
                                                               const float* __restrict__ alpha, int n, int m, int n_sample,
                                                               float* __restrict__ weight) {
  const int s = blockIdx.x * blockDim.x + threadIdx.x;
  const int sc = s < n_sample ? s : n_sample - 1;
  uint32_t covered = 0;
  for (int i = 0; i < n; ++i) {
    uint64_t all = ~0ull;
    for (int k = 0; k < m; ++k)
      all &= __builtin_amdgcn_ballot_w64(fit_t[(int64_t)k * n + i] <= samples_t[(int64_t)k * n_sample + sc]);
    covered += (uint32_t)((all >> (threadIdx.x & 63)) & 1ull);
  }
  if (s < n_sample) weight[s] = alpha[covered == 0u ? 0 : covered - 1u];
}

// partial[chunk][i] = sum over the samples s of the chunk, in ascending s, of (pds[s, i] ? weight[s] : 0);
// lane = point, samples stream past.  grid = (point blocks, chunks).
__global__ __launch_bounds__(256) void hv_point_partial_kernel(const float* __restrict__ fit_t, const float* __restrict__ samples_t,
                                                               const float* __restrict__ weight, int n, int m, int n_sample,
                                                               float* __restrict__ partial) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  const int ic = i < n ? i : n - 1;
  const int s_begin = blockIdx.y * kHvChunk;
  const int s_end = min(n_sample, s_begin + kHvChunk);
  float acc = 0.0f;
  for (int s = s_begin; s < s_end; ++s) {
    uint64_t all = ~0ull;
    for (int k = 0; k < m; ++k)
      all &= __builtin_amdgcn_ballot_w64(fit_t[(int64_t)k * n + ic] <= samples_t[(int64_t)k * n_sample + s]);
    const float w = weight[s];
    acc += ((all >> (threadIdx.x & 63)) & 1ull) ? w : 0.0f;
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

}  // namespace evx
