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

// (see the kernels that order a last front without sorting the costs, below)
constexpr int kWideDirectRows = 24576;
// Beyond a front of this many rows the sorts are the faster way (direct: 160 us at 8192 candidates of three objectives,
// 950 at 20 000); the host goes by what the last selection of the shape found (`outcome`: pinned host memory or
// null; 1 = a front up to this size, 2 = a larger one), and either way handles a front of any size.
constexpr int kWideDirectFront = 8192;

struct WideCtrl {
  int nv;     // rows selected by the mask
  int worst;  // with a rank vector: the largest rank that is not EVOX_HIP_RANK_UNSET (the mask is rank == worst)
  int err;    // an order came back poisoned (a sort's bounded device-side wait ran out): the results are poisoned too
  int start;  // with a rank vector: the rows of the fronts before that one
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
// blockIdx.z: one of several populations (rank vectors n entries apart, control blocks ws_step bytes apart).
__global__ __launch_bounds__(1024) void wide_head_kernel(const uint8_t* __restrict__ mask, int64_t mask_stride,
                                                         const int* __restrict__ rank, int n, WideCtrl* __restrict__ ctrl,
                                                         int64_t ws_step = 0) {
  __shared__ int red[16];
  if (rank != nullptr) rank += (int64_t)blockIdx.z * n;
  ctrl = reinterpret_cast<WideCtrl*>(reinterpret_cast<char*>(ctrl) + (int64_t)blockIdx.z * ws_step);
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
  int count = 0, better = 0;
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    count += rank != nullptr ? (rank[i] == worst) : (mask != nullptr ? (mask[(int64_t)i * mask_stride] != 0) : 1);
    better += rank != nullptr && rank[i] < worst ? 1 : 0;
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    count += __shfl_xor(count, off);
    better += __shfl_xor(better, off);
  }
  __shared__ int red_better[16];
  if (lane == 0) {
    red[wave] = count;
    red_better[wave] = better;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int v = 1; v < (int)(blockDim.x >> 6); ++v) {
      count += red[v];
      better += red_better[v];
    }
    ctrl->nv = count;
    ctrl->worst = worst;
    ctrl->err = 0;
    ctrl->start = better;
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
                                                       uint32_t* __restrict__ neg_hi, int* __restrict__ outcome) {
  const bool failed = ctrl->err != 0;
  if (outcome != nullptr && blockIdx.x == 0 && threadIdx.x == 0)
    __hip_atomic_store(outcome, ctrl->nv > kWideDirectFront ? 2 : 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
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

// ---- The same distances and the selection order without a sort of the costs, for populations of up to
// kWideDirectRows rows.  `listing` holds the rows by (rank, row index) -- one stable argsort step of the ranks -- so
// the rows of the last front are listing[start .. start + nv) in index order: candidate q of the front.  A candidate's
// neighbours in an objective's order (non_dominate.py:221-225: by cost, ties by row index) are the largest composite
// (ordered image of the cost, candidate number) below its own and the smallest above; sixteen lanes look for them
// among all candidates, as crowd_small_front (finish.hpp) does for 4-byte costs held in LDS.  The work grows with the
// square of the front -- 10 us for a front of some hundred rows, where the sorts of all n rows by every objective take
// twelve launches of 40 us at 20 000 rows, and about as long as those sorts when all 20 000 rows are one front.

__device__ inline uint64_t wide_image(const void* costs, int kind, int64_t at) {
  return kind == kWideFloat64   ? ordered_key64(static_cast<const double*>(costs)[at])
         : kind == kWideFloat32 ? ordered_key64((double)static_cast<const float*>(costs)[at])
                                : ordered_key64(static_cast<const long long*>(costs)[at]);
}

// key[k][q] (columns n apart) of every candidate; dist = -inf for every row (the candidates' are written afterwards);
// and, by workgroup k < m (or every gridDim.x-th objective), the candidates that stand first and last in objective
// k's order: ends[2k], ends[2k + 1].
template <class Out>
__global__ __launch_bounds__(256) void wide_front_keys_kernel(const void* __restrict__ costs, int kind, int64_t stride_row,
                                                              int64_t stride_col, int n, int m, const int* __restrict__ listing,
                                                              const WideCtrl* __restrict__ ctrl, uint64_t* __restrict__ key,
                                                              int* __restrict__ ends, Out* __restrict__ dist, int64_t ws_step = 0,
                                                              int64_t cost_step = 0) {
  __shared__ uint64_t lo_key[4], hi_key[4];
  // (blockIdx.z: one of several populations, their buffers ws_step bytes and their costs cost_step bytes apart)
  to_population(ws_step, listing, ctrl, key, ends, dist);
  costs = static_cast<const char*>(costs) + (int64_t)blockIdx.z * cost_step;
  __shared__ int lo_at[4], hi_at[4];
  const int nv = ctrl->nv, start = ctrl->start;
  for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) dist[i] = (Out)(-INFINITY);
  const int64_t total = (int64_t)nv * m;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * blockDim.x) {
    const int k = (int)(idx / nv), q = (int)(idx - (int64_t)k * nv);
    const int row = listing[start + q];
    key[(int64_t)k * n + q] = row < 0 ? ~0ull : wide_image(costs, kind, (int64_t)row * stride_row + (int64_t)k * stride_col);
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int k = blockIdx.x; k < m; k += gridDim.x) {
    uint64_t lo = ~0ull, hi = 0ull;
    int lo_q = -1, hi_q = -1;  // (ascending q per thread: the first of equal images stays first, the last one last)
    for (int q = threadIdx.x; q < nv; q += blockDim.x) {
      const int row = listing[start + q];
      const uint64_t image = row < 0 ? ~0ull : wide_image(costs, kind, (int64_t)row * stride_row + (int64_t)k * stride_col);
      if (lo_q < 0 || image < lo) lo = image, lo_q = q;
      if (hi_q < 0 || image >= hi) hi = image, hi_q = q;
    }
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const uint64_t other_lo = ((uint64_t)__shfl_xor((unsigned)(lo >> 32), off) << 32) | (unsigned)__shfl_xor((unsigned)lo, off);
      const uint64_t other_hi = ((uint64_t)__shfl_xor((unsigned)(hi >> 32), off) << 32) | (unsigned)__shfl_xor((unsigned)hi, off);
      const int other_lo_q = __shfl_xor(lo_q, off), other_hi_q = __shfl_xor(hi_q, off);
      if (other_lo_q >= 0 && (lo_q < 0 || other_lo < lo || (other_lo == lo && other_lo_q < lo_q))) lo = other_lo, lo_q = other_lo_q;
      if (other_hi_q >= 0 && (hi_q < 0 || other_hi > hi || (other_hi == hi && other_hi_q > hi_q))) hi = other_hi, hi_q = other_hi_q;
    }
    __syncthreads();  // (the arrays are reused from objective to objective)
    if (lane == 0) {
      lo_key[wave] = lo;
      lo_at[wave] = lo_q;
      hi_key[wave] = hi;
      hi_at[wave] = hi_q;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
      for (int v = 1; v < (int)(blockDim.x >> 6); ++v) {
        if (lo_at[v] >= 0 && (lo_q < 0 || lo_key[v] < lo || (lo_key[v] == lo && lo_at[v] < lo_q))) lo = lo_key[v], lo_q = lo_at[v];
        if (hi_at[v] >= 0 && (hi_q < 0 || hi_key[v] > hi || (hi_key[v] == hi && hi_at[v] > hi_q))) hi = hi_key[v], hi_q = hi_at[v];
      }
      ends[2 * k] = lo_q;
      ends[2 * k + 1] = hi_q;
    }
  }
}

// The distance of every candidate (written by row) and the ordered image of its negative (by candidate number).
// Grid: a group of sixteen lanes per row of the population (ceil(n / 16) workgroups of 256 threads); the groups
// beyond the front have nothing to do.  A front of up to kWideStagedFront rows has the images of an objective staged in
// the LDS of every workgroup that holds candidates (otherwise every step of the search is a round trip to the L2:
// 25 us for a front of 600 rows).
constexpr int kWideStagedFront = 4096;

template <class Out>
__global__ __launch_bounds__(256) void wide_front_dist_kernel(const void* __restrict__ costs, int kind, int64_t stride_row,
                                                              int64_t stride_col, int n, int m, const int* __restrict__ listing,
                                                              WideCtrl* __restrict__ ctrl, const uint64_t* __restrict__ key,
                                                              const int* __restrict__ ends, Out* __restrict__ dist,
                                                              uint64_t* __restrict__ dkey, int64_t ws_step = 0,
                                                              int64_t cost_step = 0) {
  __shared__ uint64_t staged[kWideStagedFront];
  to_population(ws_step, listing, ctrl, key, ends, dist, dkey);
  costs = static_cast<const char*>(costs) + (int64_t)blockIdx.z * cost_step;
  const int nv = ctrl->nv, start = ctrl->start;
  if ((int)(blockIdx.x * (blockDim.x >> 4)) >= nv) return;  // (the whole workgroup)
  const int sub = threadIdx.x & 15;
  const int q = (int)(blockIdx.x * (blockDim.x >> 4) + (threadIdx.x >> 4));
  const bool mine_exists = q < nv;
  const bool stage = nv <= kWideStagedFront;
  const int row = mine_exists ? listing[start + q] : -1;
  bool boundary = false;
  Out acc = (Out)0;
  for (int k = 0; k < m; ++k) {
    const uint64_t* __restrict__ col = key + (int64_t)k * n;
    if (stage) {
      __syncthreads();  // (the searches of the objective before are over)
      for (int e = threadIdx.x; e < nv; e += blockDim.x) staged[e] = col[e];
      __syncthreads();
    }
    if (!mine_exists) continue;
    const uint64_t mine = stage ? staged[q] : col[q];
    uint64_t below = 0ull, above = ~0ull;
    int below_q = -1, above_q = -1;
    for (int e0 = sub; e0 < nv; e0 += 4 * 16) {  // four partners per step, their loads in flight together
      uint64_t c[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) c[u] = e0 + 16 * u < nv ? (stage ? staged[e0 + 16 * u] : col[e0 + 16 * u]) : mine;
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int e = e0 + 16 * u;  // (e ascends within a lane)
        const bool before = c[u] < mine || (c[u] == mine && e < q);
        const bool after = c[u] > mine || (c[u] == mine && e > q);
        if (e < nv && before && (below_q < 0 || c[u] >= below)) below = c[u], below_q = e;  // the last of the largest
        if (e < nv && after && (above_q < 0 || c[u] < above)) above = c[u], above_q = e;    // the first of the smallest
      }
    }
#pragma unroll
    for (int off = 1; off < 16; off <<= 1) {
      const uint64_t ob = ((uint64_t)__shfl_xor((unsigned)(below >> 32), off) << 32) | (unsigned)__shfl_xor((unsigned)below, off);
      const uint64_t oa = ((uint64_t)__shfl_xor((unsigned)(above >> 32), off) << 32) | (unsigned)__shfl_xor((unsigned)above, off);
      const int obq = __shfl_xor(below_q, off), oaq = __shfl_xor(above_q, off);
      if (obq >= 0 && (below_q < 0 || ob > below || (ob == below && obq > below_q))) below = ob, below_q = obq;
      if (oaq >= 0 && (above_q < 0 || oa < above || (oa == above && oaq < above_q))) above = oa, above_q = oaq;
    }
    if (below_q < 0 || above_q < 0) {
      boundary = true;  // first or last of this objective (non_dominate.py:226-227)
    } else if (row >= 0) {
      const int64_t c0 = (int64_t)k * stride_col;
      const Out term = wide_term<Out>(costs, kind, (int64_t)listing[start + above_q] * stride_row + c0,
                                      (int64_t)listing[start + below_q] * stride_row + c0,
                                      (int64_t)listing[start + ends[2 * k + 1]] * stride_row + c0,
                                      (int64_t)listing[start + ends[2 * k]] * stride_row + c0);
      acc = k == 0 ? term : acc + term;
    }
  }
  if (mine_exists && sub == 0) {
    if (row < 0) {  // a poisoned listing
      ctrl->err = 1;
      dkey[q] = ~0ull;
    } else {
      const Out d = boundary ? (Out)INFINITY : acc;
      dist[row] = d;
      dkey[q] = ordered_key64(-(double)d);
    }
  }
}

// The selection order: the fronts before the last one as listed, the candidates by (distance descending, NaN last,
// row index), what the ranking left without a rank behind them as listed.  Every entry -1 when something was poisoned.
__global__ __launch_bounds__(256) void wide_front_order_kernel(const int* __restrict__ listing, const WideCtrl* __restrict__ ctrl,
                                                               const uint64_t* __restrict__ dkey, int n, int* __restrict__ order,
                                                               int* __restrict__ outcome, int64_t ws_step = 0) {
  to_population(ws_step, listing, ctrl, dkey, order);
  const int nv = ctrl->nv, start = ctrl->start;
  const bool failed = ctrl->err != 0;
  if (outcome != nullptr && blockIdx.x == 0 && blockIdx.z == 0 && threadIdx.x == 0)
    __hip_atomic_store(outcome, nv > kWideDirectFront ? 2 : 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
  for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x)
    if (failed)
      order[i] = -1;
    else if (i < start || i >= start + nv)
      order[i] = listing[i];
  if (failed) return;
  const int sub = threadIdx.x & 15;
  const int groups = (int)(gridDim.x * (blockDim.x >> 4));
  for (int q = (int)(blockIdx.x * (blockDim.x >> 4) + (threadIdx.x >> 4)); q < nv; q += groups) {
    const uint64_t mine = dkey[q];
    int smaller = 0;
    for (int e0 = sub; e0 < nv; e0 += 4 * 16) {
      uint64_t c[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) c[u] = e0 + 16 * u < nv ? dkey[e0 + 16 * u] : ~0ull;
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int e = e0 + 16 * u;
        smaller += e < nv && (c[u] < mine || (c[u] == mine && e < q)) ? 1 : 0;
      }
    }
#pragma unroll
    for (int off = 1; off < 16; off <<= 1) smaller += __shfl_xor(smaller, off);
    if (sub == 0) order[start + smaller] = listing[start + q];
  }
}

// ---- The dense ranks of the values of one objective, from their sorted order: what the ranking kernels, which read
// 4-byte floats, get in place of 8-byte fitness (dominance only looks at the order of the values inside an objective).
// One workgroup per sorted row: sorted[row][p] ascending (NaN last), index[row][p] the place the value came from;
// out[(b * n + index) * m + k] for row = b * m + k gets the number of distinct values before it (-0.0 and 0.0 are one
// value), as a float -- exact below 2^24 -- and NaN where the value is NaN.
constexpr int kDenseRankThreads = 1024;
constexpr int kDenseRankPer = 16;  // (four: 25 us for 20 000 values a row, the passes over 4096 values each being chains of barriers; sixteen: see below)

template <class T>
__global__ __launch_bounds__(kDenseRankThreads) void dense_rank_kernel(const T* __restrict__ sorted, const int64_t* __restrict__ index,
                                                                       int n, int m, float* __restrict__ out) {
  __shared__ int wave_total[kDenseRankThreads / 64];
  __shared__ int carry_lds;
  const int row = blockIdx.x, b = row / m, k = row - b * m;
  const T* __restrict__ v = sorted + (int64_t)row * n;
  const int64_t* __restrict__ at = index + (int64_t)row * n;
  float* __restrict__ dst = out + (int64_t)b * n * m + k;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (threadIdx.x == 0) carry_lds = 0;
  __syncthreads();
  for (int base = 0; base < n; base += kDenseRankThreads * kDenseRankPer) {
    const int p0 = base + (int)threadIdx.x * kDenseRankPer;
    int opens[kDenseRankPer];
    T mine[kDenseRankPer];
    T before = p0 > 0 && p0 - 1 < n ? v[p0 - 1] : T(0);
    int sum = 0;
#pragma unroll
    for (int e = 0; e < kDenseRankPer; ++e) {
      const int p = p0 + e;
      mine[e] = p < n ? v[p] : T(0);
      opens[e] = p > 0 && p < n && mine[e] != before ? 1 : 0;  // (a NaN differs from everything, itself included)
      sum += opens[e];
      before = mine[e];
    }
    int incl = sum;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const int up = __shfl_up(incl, off);
      if (lane >= off) incl += up;
    }
    if (lane == 63) wave_total[wave] = incl;
    __syncthreads();
    int rank = carry_lds + incl - sum;
    for (int w = 0; w < wave; ++w) rank += wave_total[w];
#pragma unroll
    for (int e = 0; e < kDenseRankPer; ++e) {
      const int p = p0 + e;
      rank += opens[e];
      if (p < n) dst[at[p] * m] = mine[e] != mine[e] ? NAN : (float)rank;
    }
    __syncthreads();
    if (threadIdx.x == kDenseRankThreads - 1) carry_lds = rank;  // (the last thread's last rank: everything so far)
    __syncthreads();
  }
}

// Up to four gathers of rows by one order in one launch (decision vectors, fitness rows, ranks, distances of a
// selection): dst row r = src row order[r] (raw bytes) for r < count, unit[p] bytes at a time; all-ones bytes for a row
// of a poisoned order (-1).  Part p copies rows of row_bytes[p] bytes.
struct GatherParts {
  const uint8_t* src[4];
  uint8_t* dst[4];
  int64_t row_bytes[4], row_stride_bytes[4];
  int64_t first[5];  // the work items (count x units per row) of part p are first[p] .. first[p + 1]
  int64_t src_step[4], dst_step[4];  // several populations in the launch (blockIdx.z): bytes from one to the next
  int unit[4];
  int parts;
};

__global__ __launch_bounds__(256) void gather_parts_kernel(GatherParts g, const int* __restrict__ order, int64_t count,
                                                           int64_t order_step = 0) {
  order = reinterpret_cast<const int*>(reinterpret_cast<const char*>(order) + (int64_t)blockIdx.z * order_step);
  for (int p = 0; p < g.parts; ++p) {
    g.src[p] += (int64_t)blockIdx.z * g.src_step[p];
    g.dst[p] += (int64_t)blockIdx.z * g.dst_step[p];
  }
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < g.first[g.parts]; idx += (int64_t)gridDim.x * blockDim.x) {
    int p = 0;
    while (p + 1 < g.parts && idx >= g.first[p + 1]) ++p;
    const int unit = g.unit[p];
    const int64_t per_row = g.row_bytes[p] / unit;
    const int64_t local = idx - g.first[p];
    const int64_t r = local / per_row, u = local - r * per_row;
    const int row = order[r];
    uint8_t* to = g.dst[p] + r * g.row_bytes[p] + u * unit;
    if (row < 0) {
      for (int b = 0; b < unit; ++b) to[b] = 0xFF;
      continue;
    }
    const uint8_t* from = g.src[p] + (int64_t)row * g.row_stride_bytes[p] + u * unit;
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
