// Non-domination ranks of a population of TWO objectives without a dominance matrix.
//
// Reference semantics (src/evox/operators/selection/non_dominate.py:6-26, :161-195): row i dominates row j when it is
// no worse in both objectives and the rows differ; rank r is the front of what remains after the fronts before it.
// With two objectives the relation is a staircase.  Sort the rows by (first objective, second objective, index) --
// the slot sort of order.hpp on the key (image of f1) << 32 | image of f2, which also finds the rows that are
// identical (equal keys: they get the rank of the first of them and never count against each other).  Every
// dominator of a row then stands before it, and a row is dominated by an earlier one exactly when that row's second
// objective is no larger: the front of what remains is the set of strict prefix minima of the second objective.
// Each round of the peeling is therefore one prefix-minimum scan, O(n) work and no n^2 anywhere, where the matrix
// formulation pays n^2 / 2 pair tests and a pass over bit rows per front (two objectives give many thin fronts:
// 380 of them at 200 000 rows).
//
// The scan of a round runs through the workgroups like a bucket brigade: workgroup b owns a run of slots, receives
// the minimum over the remaining rows before its run from workgroup b - 1, hands min(that, its own minimum) on to
// workgroup b + 1 AT ONCE -- before its own scan -- and then ranks its rows.  A round costs a workgroup one scan in
// registers and LDS, and the rounds of different workgroups overlap: F fronts over B workgroups take about F + B
// hand-overs, not F * B.  A workgroup only ever waits for the one before it (and, when it is a whole ring of rounds
// ahead, for the one after it); all waits are bounded.  Rows holding a NaN neither dominate nor are dominated: rank 0,
// and they take no part.
#pragma once

#include "peel.hpp"

namespace evx {

// (256 threads x 16 slots, one wave per SIMD, was slower: 1.5 against 0.75 us per round -- the running minimum over a
// thread's own slots is a chain of dependent instructions that no other wave hides.)
constexpr int kTwoThreads = 1024;
constexpr int kTwoPerThread = 4;                             // consecutive slots per thread
constexpr int kTwoChunk = kTwoThreads * kTwoPerThread;       // slots per workgroup
constexpr int kTwoMaxBlocks = 256;
constexpr int64_t kTwoMaxRows = (int64_t)kTwoChunk * kTwoMaxBlocks;
constexpr int kTwoRing = 256;                                // rounds of a workgroup's outgoing stream that are kept
constexpr int kTwoRingStride = kTwoRing + 16;                // words per workgroup: the ring, then its progress counter on a line of its own
constexpr uint32_t kTwoNone = 0xFFFFFFFFu;                   // "no remaining row": larger than every image of a number
constexpr unsigned kTwoEnd = 0x80000000u;                    // in a word's tag: nothing remains in this workgroup or before it

// Inclusive prefix minimum over the lanes of a wave (DPP row shifts and row broadcasts).
__device__ inline uint32_t wave_prefix_min(uint32_t x) {
  uint32_t v = x;
  v = min(v, (uint32_t)__builtin_amdgcn_update_dpp((int)kTwoNone, (int)x, 0x111, 0xf, 0xf, false));  // row_shr:1
  v = min(v, (uint32_t)__builtin_amdgcn_update_dpp((int)kTwoNone, (int)x, 0x112, 0xf, 0xf, false));  // row_shr:2
  v = min(v, (uint32_t)__builtin_amdgcn_update_dpp((int)kTwoNone, (int)x, 0x113, 0xf, 0xf, false));  // row_shr:3
  v = min(v, (uint32_t)__builtin_amdgcn_update_dpp((int)kTwoNone, (int)v, 0x114, 0xf, 0xe, false));  // row_shr:4
  v = min(v, (uint32_t)__builtin_amdgcn_update_dpp((int)kTwoNone, (int)v, 0x118, 0xf, 0xc, false));  // row_shr:8
  v = min(v, (uint32_t)__builtin_amdgcn_update_dpp((int)kTwoNone, (int)v, 0x142, 0xa, 0xf, false));  // row_bcast:15
  v = min(v, (uint32_t)__builtin_amdgcn_update_dpp((int)kTwoNone, (int)v, 0x143, 0xc, 0xf, false));  // row_bcast:31
  return v;
}

// Grid: ceil(n / kTwoChunk) workgroups of kTwoThreads.  xs1_sorted / xs2_sorted: the objectives by slot (rows sorted by
// (f1, f2, index)); kid: first slot of the slot's key.  Writes the rank of every row that is the first of its key
// (by original index), rank 0 for rows holding a NaN, and the -inf fill of the distances; every front is peeled.
// ring: gridDim.x * kTwoRingStride words, zero at the start of the call.
__global__ __launch_bounds__(kTwoThreads) void two_peel_kernel(const float* __restrict__ xs1_sorted, const float* __restrict__ xs2_sorted,
                                                               const uint32_t* __restrict__ kid, const int* __restrict__ orig_of,
                                                               int n, int* __restrict__ rank, float* __restrict__ dist_fill,
                                                               Ctrl* __restrict__ ctrl, unsigned long long* __restrict__ ring,
                                                               unsigned spin_limit) {
  __shared__ __attribute__((aligned(16))) uint32_t wave_min_lds[2][kTwoThreads / 64];  // by the parity of the round: a wave may be a round ahead of another's reads
  __shared__ uint32_t in_lds[2];  // the round's incoming minimum; 1 when the workgroup leaves after this round's hand-over
  __shared__ uint32_t before_lds[kTwoThreads / 64];  // the minimum over the waves before each wave
  __shared__ int ranked_lds;      // rows this workgroup ranked in the round
  if (coherent_load(&ctrl->err) != 0) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int b = blockIdx.x;
  const bool last_block = b == (int)gridDim.x - 1;
  unsigned long long* my_ring = ring + (size_t)b * kTwoRingStride;
  const unsigned long long* up_ring = ring + (size_t)(b > 0 ? b - 1 : 0) * kTwoRingStride;
  int* my_progress = reinterpret_cast<int*>(my_ring + kTwoRing);  // rounds of the stream before that this workgroup has taken in
  const int* down_progress = reinterpret_cast<const int*>(ring + (size_t)(last_block ? b : b + 1) * kTwoRingStride + kTwoRing);
  // ---- this thread's slots
  uint32_t v[kTwoPerThread];
  int orig[kTwoPerThread];
  int unranked = 0;
  {
    const int s0 = b * kTwoChunk + tid * kTwoPerThread;
#pragma unroll
    for (int e = 0; e < kTwoPerThread; ++e) {
      const int s = s0 + e;
      v[e] = kTwoNone;
      orig[e] = 0;
      if (s < n) {
        const float a1 = xs1_sorted[s], a2 = xs2_sorted[s];
        const int o = orig_of[s];
        if (dist_fill) dist_fill[o] = -INFINITY;
        if (a1 != a1 || a2 != a2) {
          rank[o] = 0;  // a row holding a NaN neither dominates nor is dominated (every comparison is false, non_dominate.py:20-24)
        } else if (kid[s] == (uint32_t)s) {
          v[e] = ordered_key(a2);
          orig[e] = o;
          ++unranked;
        }  // (the other rows of a key take the rank of its first row afterwards: two_finish_kernel)
      }
    }
  }
  if (tid == 0) ranked_lds = 0;
  unranked = wave_sum(unranked);
  if (lane == 0) wave_min_lds[1][wave] = (uint32_t)unranked;
  __syncthreads();
  int left = 0;  // (thread 0 keeps the count of this workgroup's unranked rows)
  if (tid == 0)
    for (int w = 0; w < kTwoThreads / 64; ++w) left += (int)wave_min_lds[1][w];
  __syncthreads();
  bool upstream_ended = b == 0;
  // (thread 0) the words of the next two rounds are asked for ahead of time: the workgroup before is usually a round
  // or more ahead, so that a round finds its word there and pays no memory round trip
  unsigned long long ahead[2] = {0ull, 0ull};
  if (tid == 0 && !upstream_ended) {
    ahead[0] = coherent_load(up_ring + 0);
    ahead[1] = coherent_load(up_ring + (1 % kTwoRing));
  }
  for (int round = 0;; ++round) {
    const unsigned tag = (unsigned)round + 1u;
    // ---- the minimum of this workgroup's remaining rows
    uint32_t tmin = kTwoNone;
#pragma unroll
    for (int e = 0; e < kTwoPerThread; ++e) tmin = min(tmin, v[e]);
    const uint32_t incl = wave_prefix_min(tmin);
    uint32_t* const wave_min = wave_min_lds[round & 1];
    if (lane == 63) wave_min[wave] = incl;
    EVX_TRACE(round, 0);
    lds_barrier();
    EVX_TRACE(round, 1);
    // the first wave turns the wave minima into what stands before every wave (a prefix minimum over sixteen lanes
    // of a DPP row) and the minimum of the workgroup
    uint32_t local = kTwoNone;
    if (wave == 0) {
      const uint32_t mine = lane < kTwoThreads / 64 ? wave_min[lane] : kTwoNone;
      const uint32_t upto = wave_prefix_min(mine);
      const uint32_t before_wave = (uint32_t)__builtin_amdgcn_update_dpp((int)kTwoNone, (int)upto, 0x138, 0xf, 0xf, false);  // wave_shr:1
      if (lane < kTwoThreads / 64) before_lds[lane] = before_wave;
      local = (uint32_t)__builtin_amdgcn_readlane((int)upto, kTwoThreads / 64 - 1);
    }
    if (tid == 0) {
      left -= ranked_lds;  // what the round before has ranked
      ranked_lds = 0;
      // ---- the incoming minimum of the round
      uint32_t in = kTwoNone;
      bool failed = false;
      if (!upstream_ended) {
        const unsigned long long* slot = up_ring + (round % kTwoRing);
        unsigned long long word = ahead[0];
        ahead[0] = ahead[1];
        if (((unsigned)(word >> 32) & ~kTwoEnd) != tag) {
          WaitBound bound(spin_limit);
          for (unsigned spins = 0;; ++spins) {
            word = coherent_load(slot);
            if (((unsigned)(word >> 32) & ~kTwoEnd) == tag) break;
            if (bound.expired(spins) || ((spins & 63u) == 63u && coherent_load(&ctrl->err) != 0)) {
              failed = true;
              break;
            }
          }
        }
        if (!failed) {
          in = (uint32_t)word;
          if ((unsigned)(word >> 32) & kTwoEnd) upstream_ended = true;  // nothing remains before this workgroup, from this round on
          coherent_store(my_progress, round + 1);
          if (!upstream_ended) ahead[1] = coherent_load(up_ring + ((round + 2) % kTwoRing));
        }
      }
      // ---- hand on at once: the minimum over the remaining rows up to the end of this workgroup's run.  The stream
      // ends with the round in which neither this workgroup nor those before it have a row left.
      const bool ends_here = upstream_ended && left == 0;
      if (!failed && !last_block) {
        if (round >= kTwoRing) {  // (the slot still holds round - kTwoRing: has the next workgroup taken it in?)
          WaitBound bound(spin_limit);
          for (unsigned spins = 0; coherent_load(down_progress) < round - kTwoRing + 1; ++spins) {
            if (bound.expired(spins) || ((spins & 63u) == 63u && coherent_load(&ctrl->err) != 0)) {
              failed = true;
              break;
            }
          }
        }
        if (!failed)
          coherent_store(my_ring + (round % kTwoRing), ((unsigned long long)(tag | (ends_here ? kTwoEnd : 0u)) << 32) | min(in, local));
      }
      if (failed) coherent_store(&ctrl->err, kErrBarrierTimeout);
      in_lds[0] = in;
      in_lds[1] = failed || ends_here ? 1u : 0u;
    }
    EVX_TRACE(round, 2);
    lds_barrier();
    EVX_TRACE(round, 3);
    if (in_lds[1] != 0u) break;  // nothing is left here and before, or a wait ran out
    // ---- exclusive prefix minimum over the remaining rows before each slot, seeded with the incoming one
    uint32_t before = min(in_lds[0], before_lds[wave]);
    {
      const uint32_t shifted = (uint32_t)__builtin_amdgcn_update_dpp((int)kTwoNone, (int)incl, 0x138, 0xf, 0xf, false);  // wave_shr:1
      before = min(before, shifted);
    }
    int ranked = 0;
#pragma unroll
    for (int e = 0; e < kTwoPerThread; ++e) {
      const uint32_t mine = v[e];
      if (mine < before) {  // a strict prefix minimum: no remaining row before it is no worse in both objectives
        rank[orig[e]] = round;
        v[e] = kTwoNone;
        ++ranked;
      }
      before = min(before, mine);
    }
    if (ranked) atomicAdd(&ranked_lds, ranked);  // (few threads rank a row in any one round)
    // (the barrier at the head of the next round also closes this round's counting)
  }
}

// After the brigade: the rows of a key take the rank of the key's first row.
__global__ __launch_bounds__(256) void two_finish_kernel(const uint32_t* __restrict__ kid, const int* __restrict__ orig_of,
                                                         const float* __restrict__ xs1_sorted, const float* __restrict__ xs2_sorted,
                                                         int n, int* __restrict__ rank, const Ctrl* __restrict__ ctrl) {
  if (ctrl->err != 0) return;
  for (int s = blockIdx.x * blockDim.x + threadIdx.x; s < n; s += gridDim.x * blockDim.x) {
    const int first = (int)kid[s];
    if (first == s) continue;
    const float a1 = xs1_sorted[s], a2 = xs2_sorted[s];
    if (a1 != a1 || a2 != a2) continue;  // rank 0, written by the brigade
    rank[orig_of[s]] = rank[orig_of[first]];
  }
}

// After the listing (perm = rows by (rank, original index), every row ranked, the ranks 0 .. F - 1 all present):
// where every front starts, and -- the peeling having gone through all fronts -- the front that holds the
// stop_count-th row, as the control block describes it for the kernels that order it.
__global__ __launch_bounds__(256) void two_bounds_kernel(const int* __restrict__ perm, const int* __restrict__ rank, int n,
                                                         int* __restrict__ fstart, Ctrl* __restrict__ ctrl, int stop_count) {
  if (ctrl->err != 0) return;
  const int worst = rank[perm[stop_count - 1]];
  for (int p = blockIdx.x * blockDim.x + threadIdx.x; p < n; p += gridDim.x * blockDim.x) {
    const int r = rank[perm[p]];
    const int r_before = p > 0 ? rank[perm[p - 1]] : -1;
    if (r != r_before) {  // position p opens front r
      fstart[r] = p;
      if (r == worst) {
        ctrl->worst = worst;
        ctrl->nfronts = worst + 1;
        ctrl->passes = worst;
        ctrl->worst_start = p;
        ctrl->need = stop_count - p;
      }
    }
    if (p == n - 1) fstart[r + 1] = n;
  }
}

// ... and the sizes of the fronts, from their starts (one small launch behind the one above).
__global__ __launch_bounds__(256) void two_sizes_kernel(const int* __restrict__ perm, const int* __restrict__ rank, int n,
                                                        const int* __restrict__ fstart, int* __restrict__ fsize,
                                                        Ctrl* __restrict__ ctrl, int* __restrict__ rank_until_out) {
  if (ctrl->err != 0) return;
  const int fronts = rank[perm[n - 1]] + 1;
  const int worst = ctrl->worst;
  for (int r = blockIdx.x * blockDim.x + threadIdx.x; r < fronts; r += gridDim.x * blockDim.x) {
    fsize[r] = fstart[r + 1] - fstart[r];
    if (r == worst) ctrl->nv = fstart[r + 1] - fstart[r];
  }
  // for the caller that wants the ranks only as far as that front: the rows behind it are marked unset
  if (rank_until_out != nullptr)
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) {
      const int r = rank[i];
      rank_until_out[i] = r > worst ? kRankUnset : r;
    }
}

}  // namespace evx
