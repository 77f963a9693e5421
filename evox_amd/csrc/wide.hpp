// Crowding distance and selection order for fitness of 8-byte elements (float64, int64), and -- as the tail of the
// selection path whose kernels never wait for each other (stepped.hpp) -- of float32 fitness.
//
// Reference semantics: src/evox/operators/selection/non_dominate.py:198-231 computes the distance in the dtype of the
// costs (differences) and in torch's default float dtype (the buffer that takes the quotients), so a population of
// float64 fitness under a float64 default gets float64 distances, and integer fitness gets exact integer differences
// that are divided as floats.  The kernels of the float32 path read 4-byte values; these read 8-byte ones.
//
// Division of labour: the per-objective orders (selected rows first, then cost, then row index: the lexsort of
// non_dominate.py:221) come from the stable argsort steps of radix.hpp, applied to the two 32-bit halves of an
// order-preserving 64-bit image of the cost and to the mask; the kernels here build those keys, turn the orders into
// the distance terms, add them up per row, and build the keys of the final (rank, -distance, index) order of
// non_dominate.py:253.
#pragma once

#include "common.hpp"

namespace evx {

constexpr int kWideFloat64 = 0;  // costs are IEEE doubles
constexpr int kWideInt64 = 1;    // costs are two's-complement 64-bit integers
constexpr int kWideFloat32 = 2;  // costs are IEEE floats (differences and quotients in float, as the float32 kernels compute them)

struct WideCtrl {
  int nv;     // rows selected by the mask
  int worst;  // with a rank vector: the largest rank that is not EVOX_HIP_RANK_UNSET (the mask is rank == worst)
  int err;    // an order came back poisoned (a sort's bounded device-side wait ran out): the results are poisoned too
  int pad;
};

// Order-preserving map double -> uint64 with torch's sort conventions: -0.0 and +0.0 share a key, every NaN maps to
// the largest key.
__device__ inline uint64_t ordered_key64(double v) {
  if (v != v) return ~0ull;
  uint64_t u = (uint64_t)__double_as_longlong(v);
  if (v == 0.0) u = 0ull;
  return (u >> 63) ? ~u : (u | 0x8000000000000000ull);
}
__device__ inline uint64_t ordered_key64(long long v) { return (uint64_t)v ^ 0x8000000000000000ull; }

// One workgroup: the number of selected rows, and with a rank vector the rank that selects them.
// mask: a byte per row (stride in bytes), or null; rank: int32 per row, or null (then the mask, or every row).
__global__ __launch_bounds__(1024) void wide_head_kernel(const uint8_t* __restrict__ mask, int64_t mask_stride,
                                                         const int* __restrict__ rank, int n, WideCtrl* __restrict__ ctrl) {
  __shared__ int red[16];
  __shared__ int worst_lds;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int worst = -1;
  if (rank != nullptr) {
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
      const int r = rank[i];
      if (r != kRankUnset && r > worst) worst = r;
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) worst = max(worst, __shfl_xor(worst, off));
    if (lane == 0) red[wave] = worst;
    __syncthreads();
    if (threadIdx.x == 0) {
      for (int v = 1; v < (int)(blockDim.x >> 6); ++v) worst = max(worst, red[v]);
      worst_lds = worst;
    }
    __syncthreads();
    worst = worst_lds;
    __syncthreads();
  }
  int count = 0;
  for (int i = threadIdx.x; i < n; i += blockDim.x)
    count += rank != nullptr ? (rank[i] == worst) : (mask != nullptr ? (mask[(int64_t)i * mask_stride] != 0) : 1);
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) count += __shfl_xor(count, off);
  if (lane == 0) red[wave] = count;
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int v = 1; v < (int)(blockDim.x >> 6); ++v) count += red[v];
    ctrl->nv = count;
    ctrl->worst = worst;
    ctrl->err = 0;
  }
}

// Sort keys of every (objective, row): the two halves of the cost's ordered image (key_lo / key_hi, [m][n]), the
// mask key (0 for a selected row, 1 for the others: selected rows sort first), the mask as bytes, and the cleared
// boundary flags.
__global__ __launch_bounds__(256) void wide_keys_kernel(const void* __restrict__ costs, int kind, int64_t stride_row,
                                                        int64_t stride_col, int n, int m, const uint8_t* __restrict__ mask,
                                                        int64_t mask_stride, const int* __restrict__ rank,
                                                        const WideCtrl* __restrict__ ctrl, uint32_t* __restrict__ key_lo,
                                                        uint32_t* __restrict__ key_hi, int* __restrict__ key_mask,
                                                        uint8_t* __restrict__ selected, int* __restrict__ boundary) {
  const int worst = ctrl->worst;
  const int64_t total = (int64_t)n * m;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * blockDim.x) {
    const int k = (int)(idx / n), i = (int)(idx - (int64_t)k * n);
    const int64_t at = (int64_t)i * stride_row + (int64_t)k * stride_col;
    const uint64_t image = kind == kWideFloat64   ? ordered_key64(static_cast<const double*>(costs)[at])
                           : kind == kWideFloat32 ? ordered_key64((double)static_cast<const float*>(costs)[at])
                                                  : ordered_key64(static_cast<const long long*>(costs)[at]);
    key_lo[idx] = (uint32_t)image;
    key_hi[idx] = (uint32_t)(image >> 32);
    if (k == 0) {
      const bool in = rank != nullptr ? rank[i] == worst : (mask != nullptr ? mask[(int64_t)i * mask_stride] != 0 : true);
      key_mask[i] = in ? 0 : 1;
      selected[i] = in ? 1 : 0;
      boundary[i] = 0;
    }
  }
}

template <class Out>
__device__ inline Out wide_term(const void* costs, int kind, int64_t next, int64_t prev, int64_t last, int64_t first) {
  if (kind == kWideFloat64) {
    const double* c = static_cast<const double*>(costs);
    return (Out)((c[next] - c[prev]) / (c[last] - c[first]));
  }
  if (kind == kWideFloat32) {
    const float* c = static_cast<const float*>(costs);
    return (Out)((c[next] - c[prev]) / (c[last] - c[first]));
  }
  // integers: exact differences (wrapping, as the integer subtraction of the reference), divided as floats
  const long long* c = static_cast<const long long*>(costs);
  const long long num = (long long)((unsigned long long)c[next] - (unsigned long long)c[prev]);
  const long long den = (long long)((unsigned long long)c[last] - (unsigned long long)c[first]);
  return (Out)num / (Out)den;
}

// order[k][p] = row at position p of objective k's order.  The row at an inner position gets the term
// (cost after - cost before) / (cost of the last selected row - cost of the first) of that objective
// (non_dominate.py:222-225); the rows at positions 0 and nv - 1 are flagged: they get +inf whatever their other
// terms are (:226-227).
template <class Out>
__global__ __launch_bounds__(256) void wide_terms_kernel(const void* __restrict__ costs, int kind, int64_t stride_row,
                                                         int64_t stride_col, int n, int m, const int* __restrict__ order,
                                                         WideCtrl* __restrict__ ctrl, Out* __restrict__ terms,
                                                         int* __restrict__ boundary) {
  const int nv = ctrl->nv;
  const int64_t total = (int64_t)n * m;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * blockDim.x) {
    const int k = (int)(idx / n), p = (int)(idx - (int64_t)k * n);
    const int* ord = order + (int64_t)k * n;
    const int row = ord[p];
    if (row < 0) {  // a poisoned order (all entries are -1 then)
      ctrl->err = 1;
      continue;
    }
    Out term = (Out)0;
    if (nv >= 1 && (p == 0 || p == nv - 1)) boundary[row] = 1;
    if (nv >= 1 && p >= 1 && p <= n - 2) {
      const int64_t col = (int64_t)k * stride_col;
      term = wide_term<Out>(costs, kind, (int64_t)ord[p + 1] * stride_row + col, (int64_t)ord[p - 1] * stride_row + col,
                            (int64_t)ord[nv - 1] * stride_row + col, (int64_t)ord[0] * stride_row + col);
    }
    terms[(int64_t)row * m + k] = term;
  }
}

// dist[i] = -inf outside the mask, +inf for a boundary row, else the sum of the row's terms in column order
// (non_dominate.py:228-229).  Also the two halves of the ordered image of -dist, the key of the selection order.
template <class Out>
__global__ __launch_bounds__(256) void wide_sum_kernel(const Out* __restrict__ terms, const uint8_t* __restrict__ selected,
                                                       const int* __restrict__ boundary, const WideCtrl* __restrict__ ctrl, int n,
                                                       int m, Out* __restrict__ dist, uint32_t* __restrict__ neg_lo,
                                                       uint32_t* __restrict__ neg_hi) {
  const bool failed = ctrl->err != 0;
  for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) {
    Out d;
    if (failed) {
      d = (Out)NAN;
    } else if (!selected[i]) {
      d = (Out)(-INFINITY);
    } else if (boundary[i]) {
      d = (Out)INFINITY;
    } else {
      d = terms[(int64_t)i * m];
      for (int k = 1; k < m; ++k) d += terms[(int64_t)i * m + k];
    }
    dist[i] = d;
    if (neg_lo != nullptr) {
      const uint64_t image = ordered_key64(-(double)d);  // (float -> double keeps order, infinities and NaN)
      neg_lo[i] = (uint32_t)image;
      neg_hi[i] = (uint32_t)(image >> 32);
    }
  }
}

// dst row r = src row order[r] (raw bytes), for r < count, `unit` bytes at a time; all-ones bytes for a row of a
// poisoned order (-1).
__global__ __launch_bounds__(256) void gather_rows_kernel(const uint8_t* __restrict__ src, int64_t row_bytes,
                                                          int64_t row_stride_bytes, const int* __restrict__ order, int64_t count,
                                                          uint8_t* __restrict__ dst, int unit) {
  const int64_t per_row = row_bytes / unit;
  const int64_t total = count * per_row;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = idx / per_row, u = idx - r * per_row;
    const int row = order[r];
    uint8_t* to = dst + r * row_bytes + u * unit;
    if (row < 0) {
      for (int b = 0; b < unit; ++b) to[b] = 0xFF;
      continue;
    }
    const uint8_t* from = src + (int64_t)row * row_stride_bytes + u * unit;
    if (unit == 16)
      *reinterpret_cast<uint4*>(to) = *reinterpret_cast<const uint4*>(from);
    else if (unit == 8)
      *reinterpret_cast<uint2*>(to) = *reinterpret_cast<const uint2*>(from);
    else if (unit == 4)
      *reinterpret_cast<uint32_t*>(to) = *reinterpret_cast<const uint32_t*>(from);
    else
      *to = *from;
  }
}

}  // namespace evx
