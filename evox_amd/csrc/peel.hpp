// Domination counts and front peeling over the dominated-by bit matrix.
//
// Reference semantics:
//   count[j] = sum_i A[i, j]                                   src/evox/operators/selection/non_dominate.py:188
//   front    = count == 0                                      non_dominate.py:192
//   repeat while the front is not empty (non_dominate.py:161-169):
//     rank[front] = level; count -= sum_{i in front} A[i, :]; count -= front (non_dominate.py:29-59)
//     level += 1; front = count == 0
//
// Here row j of the matrix is the dominator set of j, so count[j] = popcount(row j) and one pass
// is count[j] -= popcount(row j & front).  A row whose count reaches 0 is ranked at once and enters
// the next front; ranked rows have count 0 forever and are skipped, which is the reference's
// "count -= front" (its ranked rows sit at -1 so they never test == 0 again).
//
// The pass loop runs inside ONE persistent kernel: blocks meet at a grid barrier after every
// pass and read the size of the next front from device memory, so the host never waits for a
// front.  Block 0 does the bookkeeping of a pass while the others sweep: it lists the members of
// the current front in ascending row order into `perm` (a stable ordering by rank, which is what
// the final selection needs for every rank better than the last one) and clears the front
// buffer that the pass after next will fill.
#pragma once

#include "common.hpp"

namespace evx {

constexpr int kPeelThreads = 256;
constexpr int kRankUnset = 0x7FFFFFFF;

// Clears the control block, the front sizes and the front bitmaps (one contiguous region).
__global__ __launch_bounds__(256) void reset_state_kernel(uint32_t* __restrict__ words, int64_t n_words) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n_words; i += (int64_t)gridDim.x * blockDim.x)
    words[i] = 0u;
}

// ------------------------------------------------------------------ counts

// One wave per row: popcount of the row.  Rows with no dominator are rank 0 and form front 0.
// Also fills the crowding-distance output with -inf when one is given.
__global__ __launch_bounds__(256) void count_kernel(const uint64_t* __restrict__ dom, int64_t wstride, int nwords, int n,
                                                    int* __restrict__ count, int* __restrict__ rank,
                                                    uint64_t* __restrict__ front0, int* __restrict__ fsize,
                                                    float* __restrict__ dist_fill) {
  const int lane = threadIdx.x & 63;
  const int wave_in_block = threadIdx.x >> 6;
  const int waves = gridDim.x * (blockDim.x >> 6);
  int found = 0;
  for (int j = blockIdx.x * (blockDim.x >> 6) + wave_in_block; j < n; j += waves) {
    const uint64_t* __restrict__ row = dom + (int64_t)j * wstride;
    int c = 0;
    for (int w = lane * 2; w < nwords; w += 128) {
      const ulonglong2 v = *reinterpret_cast<const ulonglong2*>(row + w);
      c += __popcll(v.x) + __popcll(v.y);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) c += __shfl_xor(c, off);
    if (lane == 0) {
      count[j] = c;
      rank[j] = c == 0 ? 0 : kRankUnset;
      if (dist_fill) dist_fill[j] = -INFINITY;
      if (c == 0) {
        atomicOr(reinterpret_cast<unsigned long long*>(front0 + (j >> 6)), 1ull << (j & 63));
        ++found;
      }
    }
  }
  if (lane == 0 && found) atomicAdd(fsize, found);
}

// ------------------------------------------------------------ grid barrier

// Relaxed agent-scope accesses: they go to the level that all XCDs share (each XCD has an L2 of
// its own), one location at a time, without the whole-cache write-back / invalidate that an
// agent-scope fence costs.  Everything that one block writes and another block reads during the
// kernel (front bitmaps, front sizes, barrier flags) is accessed only through these.
template <class T>
__device__ inline T coherent_load(const T* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
template <class T>
__device__ inline void coherent_store(T* p, T v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Flag-array barrier: every block publishes the generation in its own slot, block 0 waits for all
// slots and then publishes the generation in `release`, the others wait for that.  No
// read-modify-write contention.  __syncthreads() makes every wave wait for its own outstanding
// memory operations (it carries a workgroup-scope fence) before the block's flag is written, and
// the data exchanged across the barrier is accessed coherently (see above), so no cache-wide fence
// is needed.  Every wait is bounded by `spin_limit` polls, after which the error flag is set and the
// caller leaves its loop, so all waves always finish.
__device__ inline bool grid_barrier(Ctrl* ctrl, unsigned gen, unsigned spin_limit) {
  __syncthreads();
  if (blockIdx.x == 0) {
    bool ok = true;
    for (unsigned b = 1 + threadIdx.x; b < gridDim.x; b += blockDim.x) {
      unsigned spins = 0;
      while (coherent_load(&ctrl->arrive[b]) < gen) {
        if (++spins > spin_limit) {
          ok = false;
          break;
        }
        __builtin_amdgcn_s_sleep(1);
      }
    }
    if (!ok) coherent_store(&ctrl->err, kErrBarrierTimeout);
    __syncthreads();
    if (threadIdx.x == 0) coherent_store(&ctrl->release, gen);
  } else {
    if (threadIdx.x == 0) {
      coherent_store(&ctrl->arrive[blockIdx.x], gen);
      unsigned spins = 0;
      while (coherent_load(&ctrl->release) < gen) {
        if (++spins > spin_limit) {
          coherent_store(&ctrl->err, kErrBarrierTimeout);
          break;
        }
        __builtin_amdgcn_s_sleep(1);
      }
    }
  }
  __syncthreads();
  return coherent_load(&ctrl->err) == 0;
}

// -------------------------------------------------------------- one sweep

// count[j] -= popcount(row j & front) for every row of this wave's share that is still unranked.
// `front_lds` is the current front copied to LDS.  Returns the number of rows this thread moved
// into the next front (non-zero on lane 0 only).
__device__ inline int sweep_rows(const uint64_t* __restrict__ dom, int64_t wstride, int nwords, int n,
                                 const uint64_t* front_lds, int* __restrict__ count, int* __restrict__ rank,
                                 uint64_t* __restrict__ next_front, int next_level, int first_row, int row_step) {
  const int lane = threadIdx.x & 63;
  int found = 0;
  for (int j = first_row; j < n; j += row_step) {
    const int cj = count[j];  // wave-uniform
    if (cj <= 0) continue;
    const uint64_t* __restrict__ row = dom + (int64_t)j * wstride;
    int c = 0;
    for (int w = lane * 2; w < nwords; w += 128) {
      const ulonglong2 v = *reinterpret_cast<const ulonglong2*>(row + w);
      c += __popcll(v.x & front_lds[w]) + __popcll(v.y & front_lds[w + 1]);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) c += __shfl_xor(c, off);
    if (lane == 0 && c) {
      const int left = cj - c;
      count[j] = left;
      if (left == 0) {
        rank[j] = next_level;
        atomicOr(reinterpret_cast<unsigned long long*>(next_front + (j >> 6)), 1ull << (j & 63));
        ++found;
      }
    }
  }
  return found;
}

// Block-wide listing of the set bits of `front` (nwords words, LDS) in ascending order into
// perm[base ...].  `scratch` holds blockDim.x ints.
__device__ inline void list_front(const uint64_t* front_lds, int nwords, int* __restrict__ perm, int base, int* scratch) {
  // each thread owns a contiguous slice of words so that the order is ascending
  const int per = (nwords + blockDim.x - 1) / blockDim.x;
  const int w_begin = threadIdx.x * per;
  const int w_end = min(nwords, w_begin + per);
  int mine = 0;
  for (int w = w_begin; w < w_end; ++w) mine += __popcll(front_lds[w]);
  scratch[threadIdx.x] = mine;
  __syncthreads();
  // inclusive scan over blockDim.x partial sums (Hillis-Steele)
  for (int off = 1; off < (int)blockDim.x; off <<= 1) {
    const int add = threadIdx.x >= (unsigned)off ? scratch[threadIdx.x - off] : 0;
    __syncthreads();
    scratch[threadIdx.x] += add;
    __syncthreads();
  }
  int pos = base + scratch[threadIdx.x] - mine;
  for (int w = w_begin; w < w_end; ++w) {
    uint64_t bits = front_lds[w];
    while (bits) {
      const int b = __ffsll((unsigned long long)bits) - 1;
      perm[pos++] = w * 64 + b;
      bits &= bits - 1;
    }
  }
  __syncthreads();
}

// --------------------------------------------------------- persistent peel

// fronts: three buffers of nwords words (front of the pass, front being built, buffer being cleared).
// fsize[r]: size of front r (fsize[0] and fronts[0] come from count_kernel; the rest must be zero).
// perm / fstart may be null when only ranks are wanted.
// Stops as soon as the fronts listed so far hold stop_count rows (stop_count = n ranks everything).
__global__ __launch_bounds__(kPeelThreads) void peel_kernel(const uint64_t* __restrict__ dom, int64_t wstride, int nwords,
                                                             int n, int* __restrict__ count, int* __restrict__ rank,
                                                             uint64_t* __restrict__ fronts, int* __restrict__ fsize,
                                                             int* __restrict__ perm, int* __restrict__ fstart,
                                                             Ctrl* __restrict__ ctrl, int stop_count, unsigned spin_limit) {
  extern __shared__ uint64_t front_lds[];  // nwords words (nwords is even: rows are padded to 128)
  __shared__ int scratch[kPeelThreads];
  const int waves_per_block = blockDim.x >> 6;
  // block 0 keeps the books, blocks 1 .. gridDim.x-1 sweep (the host launches at least two blocks)
  const int sweep_blocks = gridDim.x - 1;
  const int sweep_block = (int)blockIdx.x - 1;
  const int row_step = sweep_blocks * waves_per_block;
  const int first_row = sweep_block * waves_per_block + (threadIdx.x >> 6);

  int level = 0;
  int ranked = 0;  // rows in fronts 0 .. level-1
  for (;;) {
    uint64_t* cur = fronts + (int64_t)(level % 3) * nwords;
    uint64_t* nxt = fronts + (int64_t)((level + 1) % 3) * nwords;
    uint64_t* old = fronts + (int64_t)((level + 2) % 3) * nwords;
    const int size = coherent_load(&fsize[level]);
    if (size <= 0) break;  // cannot happen for 1 <= stop_count <= n: a finite partial order has minimal rows
    const bool last = ranked + size >= stop_count;
    if (!last || blockIdx.x == 0) {
      for (int w = threadIdx.x; w < nwords; w += blockDim.x) front_lds[w] = coherent_load(&cur[w]);
      __syncthreads();
    }
    if (blockIdx.x == 0) {
      if (perm) list_front(front_lds, nwords, perm, ranked, scratch);
      if (threadIdx.x == 0) {
        if (fstart) fstart[level] = ranked;
        if (last) {
          if (fstart) fstart[level + 1] = ranked + size;
          ctrl->nfronts = level + 1;
          ctrl->worst = level;
          ctrl->worst_start = ranked;
          ctrl->nv = size;
          ctrl->need = stop_count - ranked;
          ctrl->passes = level;
        }
      }
      if (!last)
        for (int w = threadIdx.x; w < nwords; w += blockDim.x) coherent_store(&old[w], (uint64_t)0);
    }
    if (last) break;
    if (blockIdx.x != 0) {
      const int found = sweep_rows(dom, wstride, nwords, n, front_lds, count, rank, nxt, level + 1, first_row, row_step);
      // lane 0 of each wave holds that wave's tally: one atomic per block
      __syncthreads();
      scratch[threadIdx.x] = found;
      __syncthreads();
      if (threadIdx.x == 0) {
        int total = 0;
        for (int t = 0; t < (int)blockDim.x; t += 64) total += scratch[t];
        if (total) atomicAdd(&fsize[level + 1], total);
      }
    }
    ranked += size;
    ++level;
    if (!grid_barrier(ctrl, (unsigned)level, spin_limit)) break;
  }
}

}  // namespace evx
