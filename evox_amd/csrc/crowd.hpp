// Crowding distance over a candidate list, the index-stable top-k on the last front, and the
// fused row gather.
//
// Reference semantics:
//   crowding_distance            src/evox/operators/selection/non_dominate.py:198-231
//   lexsort (stable, last key primary)   src/evox/utils/jit_fix_operator.py:246-252
//   nd_environmental_selection   non_dominate.py:234-254
//
// The candidate list L (ascending row index, nv entries) is either the last front as listed by the
// peel kernel or the compacted mask.  Per objective k the candidates are ordered by
// (ordered_key(cost), position in L): that is torch's stable ascending sort with NaN last and signed
// zeros tied, restricted to the masked rows, which the reference puts first (non_dominate.py:215-221).
// The ordering is computed as a rank by counting, pos(q) = #{q' : (key', q') < (key, q)}: every
// candidate is compared with every other one with the partner's key coming from scalar loads, the
// same lane = row / scalar = partner structure as the dominance kernel.  The counts give the sorted
// position directly, with no passes that depend on one another.
#pragma once

#include "common.hpp"

namespace evx {

// acc += bit, the bit taken from a 64-lane mask.
__device__ inline uint32_t add_bit(uint32_t acc, uint64_t mask) {
  uint32_t r;
  uint64_t carry_out;
  asm("v_addc_co_u32_e64 %0, %1, %2, 0, %3" : "=v"(r), "=s"(carry_out) : "v"(acc), "s"(mask));
  return r;
}

// Stable compaction of a boolean mask into an ascending list (one block; n is at most a few 10^5).
// mask == nullptr selects every row.  Also fills dist with -inf and publishes nv in ctrl.
__global__ __launch_bounds__(1024) void compact_mask_kernel(const uint8_t* __restrict__ mask, int64_t mask_stride, int n,
                                                            int* __restrict__ list, float* __restrict__ dist,
                                                            Ctrl* __restrict__ ctrl) {
  __shared__ int wave_tot[16];
  __shared__ int running;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  if (threadIdx.x == 0) running = 0;
  __syncthreads();
  for (int base = 0; base < n; base += blockDim.x) {
    const int j = base + threadIdx.x;
    const bool on = j < n && (mask == nullptr || mask[j * mask_stride] != 0);
    if (j < n) dist[j] = -INFINITY;
    const uint64_t b = __builtin_amdgcn_ballot_w64(on);
    const int before = __popcll(b & ((1ull << lane) - 1ull));
    if (lane == 0) wave_tot[wave] = __popcll(b);
    __syncthreads();
    int offset = running;
    for (int w = 0; w < wave; ++w) offset += wave_tot[w];
    if (on) list[offset + before] = j;
    __syncthreads();
    if (threadIdx.x == 0) {
      int t = 0;
      for (int w = 0; w < (int)(blockDim.x >> 6); ++w) t += wave_tot[w];
      running += t;
    }
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    ctrl->worst_start = 0;
    ctrl->nv = running;
    ctrl->need = running;
  }
}

// ukey[k][q] = ordered_key(cost of candidate q in objective k); padding up to a multiple of 64 gets
// the largest key so that it never counts as smaller.  grid = (blocks over q, m).
__global__ __launch_bounds__(256) void crowd_keys_kernel(const float* __restrict__ xs, int npad, const int* __restrict__ list_base,
                                                         const Ctrl* __restrict__ ctrl, uint32_t* __restrict__ ukey,
                                                         int kstride) {
  const int nv = ctrl->nv;
  const int* __restrict__ list = list_base + ctrl->worst_start;
  const int k = blockIdx.y;
  const int nv_pad = (int)round_up(nv, 64);
  for (int q = blockIdx.x * blockDim.x + threadIdx.x; q < nv_pad; q += gridDim.x * blockDim.x)
    ukey[(int64_t)k * kstride + q] = q < nv ? ordered_key(xs[(int64_t)k * npad + list[q]]) : 0xFFFFFFFFu;
}

// pos[k][q] = sorted position of candidate q in objective k; sorted_cost[k][pos] = its cost.
// grid = (blocks over q, m); waves whose 64 candidates lie past nv leave at once.
__global__ __launch_bounds__(256) void crowd_rank_kernel(const float* __restrict__ xs, int npad, const int* __restrict__ list_base,
                                                         const Ctrl* __restrict__ ctrl, const uint32_t* __restrict__ ukey,
                                                         int kstride, int* __restrict__ pos, float* __restrict__ sorted_cost) {
  const int nv = ctrl->nv;
  const int* __restrict__ list = list_base + ctrl->worst_start;
  const int k = blockIdx.y;
  const uint32_t* __restrict__ keys = ukey + (int64_t)k * kstride;
  const int nv_pad = (int)round_up(nv, 64);
  const int waves = gridDim.x * (blockDim.x >> 6);
  const int lane = threadIdx.x & 63;
  for (int q0 = (blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6)) * 64; q0 < nv; q0 += waves * 64) {
    const int q = q0 + lane;
    const uint64_t mine = ((uint64_t)keys[q] << 32) | (uint32_t)q;  // q < nv_pad: keys are padded
    uint32_t smaller = 0;
    for (int p0 = 0; p0 < nv_pad; p0 += 8) {
#pragma unroll
      for (int t = 0; t < 8; ++t) {
        const uint64_t other = ((uint64_t)keys[p0 + t] << 32) | (uint32_t)(p0 + t);
        smaller = add_bit(smaller, __builtin_amdgcn_ballot_w64(other < mine));
      }
    }
    if (q < nv) {
      pos[(int64_t)k * kstride + q] = (int)smaller;
      sorted_cost[(int64_t)k * kstride + smaller] = xs[(int64_t)k * npad + list[q]];
    }
  }
}

// One thread per candidate: sum over objectives of (next - previous) / (last - first) in sorted
// order, +inf for a candidate that is first or last in any objective (non_dominate.py:223-229).
// Objectives are added in column order starting from the first term, which is what torch's row
// sum does for the small M of this workload.  Writes the distance of row L[q] and the key of its
// negation for the final ordering.
__global__ __launch_bounds__(256) void crowd_dist_kernel(const int* __restrict__ list_base, const Ctrl* __restrict__ ctrl, int m,
                                                         const int* __restrict__ pos, const float* __restrict__ sorted_cost,
                                                         int kstride, float* __restrict__ dist, uint32_t* __restrict__ dkey) {
  const int nv = ctrl->nv;
  const int* __restrict__ list = list_base + ctrl->worst_start;
  const int nv_pad = (int)round_up(nv, 64);
  for (int q = blockIdx.x * blockDim.x + threadIdx.x; q < nv_pad; q += gridDim.x * blockDim.x) {
    if (q >= nv) {
      if (dkey) dkey[q] = 0xFFFFFFFFu;
      continue;
    }
    bool boundary = false;
    float acc = 0.0f;
    for (int k = 0; k < m; ++k) {
      const float* __restrict__ sc = sorted_cost + (int64_t)k * kstride;
      const int p = pos[(int64_t)k * kstride + q];
      if (p == 0 || p == nv - 1) {
        boundary = true;
      } else {
        const float span = sc[nv - 1] - sc[0];
        const float term = (sc[p + 1] - sc[p - 1]) / span;
        acc = k == 0 ? term : acc + term;
      }
    }
    const float d = boundary ? INFINITY : acc;
    dist[list[q]] = d;
    if (dkey) dkey[q] = ordered_key(-d);
  }
}

// Index-stable top-k on the last front: candidate q goes to place #{q' : (dkey', q') < (dkey, q)}
// (distance descending, NaN after every number, then row index; jit_fix_operator.py:246-252 applied
// to non_dominate.py:253) and is kept when that place is below `need`.  The better fronts are copied
// from the rank-ordered listing.  grid.x covers max(n / 64 waves, copy work).
__global__ __launch_bounds__(256) void final_order_kernel(const int* __restrict__ perm, const Ctrl* __restrict__ ctrl,
                                                          const uint32_t* __restrict__ dkey, int* __restrict__ order) {
  const int nv = ctrl->nv;
  const int start = ctrl->worst_start;
  const int need = ctrl->need;
  const int* __restrict__ list = perm + start;
  const int nv_pad = (int)round_up(nv, 64);
  const int waves = gridDim.x * (blockDim.x >> 6);
  const int lane = threadIdx.x & 63;
  for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < start; i += gridDim.x * blockDim.x) order[i] = perm[i];
  for (int q0 = (blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6)) * 64; q0 < nv; q0 += waves * 64) {
    const int q = q0 + lane;
    const uint64_t mine = ((uint64_t)dkey[q] << 32) | (uint32_t)q;
    uint32_t smaller = 0;
    for (int p0 = 0; p0 < nv_pad; p0 += 8) {
#pragma unroll
      for (int t = 0; t < 8; ++t) {
        const uint64_t other = ((uint64_t)dkey[p0 + t] << 32) | (uint32_t)(p0 + t);
        smaller = add_bit(smaller, __builtin_amdgcn_ballot_w64(other < mine));
      }
    }
    if (q < nv && (int)smaller < need) order[start + smaller] = list[q];
  }
}

// out[p, :] = src[order[p], :] for the decision vectors (raw bytes, any dtype), the fitness, the rank
// and the distance.  One wave per output row; rows are copied in 16-, 4- or 1-byte units.
__global__ __launch_bounds__(256) void gather_kernel(const int* __restrict__ order, int topk, const uint8_t* __restrict__ x,
                                                     int64_t x_row_stride, int64_t x_row_bytes, uint8_t* __restrict__ out_x,
                                                     int unit, const float* __restrict__ f, int64_t f_stride_row,
                                                     int64_t f_stride_col, int m, float* __restrict__ out_f,
                                                     const int* __restrict__ rank, int* __restrict__ out_rank,
                                                     const float* __restrict__ dist, float* __restrict__ out_dist) {
  const int lane = threadIdx.x & 63;
  const int waves = gridDim.x * (blockDim.x >> 6);
  for (int p = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6); p < topk; p += waves) {
    const int64_t src = order[p];
    if (x) {
      const uint8_t* __restrict__ s = x + src * x_row_stride;
      uint8_t* __restrict__ d = out_x + (int64_t)p * x_row_bytes;
      if (unit == 16) {
        for (int64_t b = lane * 16; b < x_row_bytes; b += 64 * 16)
          *reinterpret_cast<uint4*>(d + b) = *reinterpret_cast<const uint4*>(s + b);
      } else if (unit == 4) {
        for (int64_t b = lane * 4; b < x_row_bytes; b += 64 * 4)
          *reinterpret_cast<uint32_t*>(d + b) = *reinterpret_cast<const uint32_t*>(s + b);
      } else {
        for (int64_t b = lane; b < x_row_bytes; b += 64) d[b] = s[b];
      }
    }
    for (int k = lane; k < m; k += 64) out_f[(int64_t)p * m + k] = f[src * f_stride_row + k * f_stride_col];
    if (lane == 0) {
      out_rank[p] = rank[src];
      out_dist[p] = dist[src];
    }
  }
}

}  // namespace evx
