// Segmented LSD radix sort of (32-bit key, candidate index) pairs for large fronts.
//
// Used for the per-objective ordering inside the crowding distance and for the final ordering by
// distance when the last front has more than kRadixMinCandidates rows (below that, ranking by
// counting in crowd.hpp is one pass with no dependent steps and is faster).  The result is the same
// ordering: ascending key, ties by ascending candidate index (torch's stable sort,
// src/evox/utils/jit_fix_operator.py:246-252).
//
// One persistent kernel sorts all segments together, four 8-bit passes, three grid barriers per pass
// (the barrier of peel.hpp: block 0 is the master, block 1 stays out, blocks 2.. work):
//   1. every wave histograms the digits of its contiguous share of each segment (LDS); the block
//      totals go to table[segment][digit][block];
//   2. for every (segment, digit) one wave turns the per-block counts into exclusive prefixes and
//      leaves the digit total;
//   3. every block scans the 256 digit totals, derives the first destination of each of its waves for
//      each digit, and the waves move their pairs in order: inside a group of 64 pairs the rank among
//      equal digits comes from eight ballots, so every pass is stable.
// Pairs travel between blocks through relaxed agent-scope loads and stores (no cache-wide fences).
// The sizes are read from device memory, so the host launches this unconditionally; when the front is
// small the kernel returns at once.
#pragma once

#include "common.hpp"
#include "peel.hpp"

namespace evx {

constexpr int kRadixMinCandidates = 8192;
constexpr int kRadixThreads = 256;
constexpr int kRadixBatch = 4;  // pairs per lane fetched together
constexpr int kRadixMaxWorkers = 510;  // working blocks of a radix kernel, at most (columns of the digit table)

struct RadixBuffers {
  unsigned long long* pairs[2];  // [segments][kstride] each: (key << 32) | candidate index
  int* table;                    // [segments][256][workers]
  int* totals;                   // [segments][256]
  int kstride;
};

// Sorts `nseg` segments of nv pairs; pair e of segment k is initial(k, e) (candidate order), the
// result is left in buf.pairs[0] (four passes: initial -> pairs[1] -> pairs[0] -> pairs[1] -> pairs[0]).
// Must be called by every thread of every block with blockIdx.x >= kFirstSweeper; block 0 must run
// radix_master().  `hist` = LDS, nseg * 4 * 256 ints; `base` = LDS, 256 ints.
template <class Initial>
__device__ inline bool radix_sort_segments(const RadixBuffers& buf, int nseg, int nv, Initial initial, Ctrl* ctrl,
                                           unsigned gen0, unsigned spin_limit, int* hist, int* base, int* scratch) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int workers = gridDim.x - kFirstSweeper;
  const int wb = (int)blockIdx.x - kFirstSweeper;
  const int chunk = (int)round_up((nv + workers - 1) / workers, 256);
  const int sub = chunk / 4;
  const int w_begin = min(nv, wb * chunk + wave * sub);
  const int w_end = min(nv, w_begin + sub);
  unsigned gen = gen0;
  int dummy = 0;
  for (int pass = 0; pass < 4; ++pass) {
    const int shift = 8 * pass;
    const unsigned long long* __restrict__ in = buf.pairs[pass & 1];
    unsigned long long* __restrict__ out = buf.pairs[(pass + 1) & 1];
    // ---- 1. digit histograms
    for (int t = threadIdx.x; t < nseg * 4 * 256; t += blockDim.x) hist[t] = 0;
    __syncthreads();
    // (kRadixBatch pairs per lane are fetched before any is used: the coherent loads of a wave are then in flight
    // together instead of costing a memory round trip each)
    for (int k = 0; k < nseg; ++k) {
      int* h = hist + (k * 4 + wave) * 256;
      for (int e0 = w_begin + lane; e0 < w_end; e0 += 64 * kRadixBatch) {
        unsigned long long p[kRadixBatch];
#pragma unroll
        for (int u = 0; u < kRadixBatch; ++u) {
          const int e = e0 + 64 * u;
          p[u] = e >= w_end ? 0ull : (pass == 0 ? initial(k, e) : coherent_load(&in[(int64_t)k * buf.kstride + e]));
        }
#pragma unroll
        for (int u = 0; u < kRadixBatch; ++u)
          if (e0 + 64 * u < w_end) atomicAdd(&h[(int)((p[u] >> (32 + shift)) & 255ull)], 1);
      }
    }
    __syncthreads();
    for (int k = 0; k < nseg; ++k) {
      const int d = threadIdx.x;  // blockDim.x == 256
      const int tot = hist[(k * 4 + 0) * 256 + d] + hist[(k * 4 + 1) * 256 + d] + hist[(k * 4 + 2) * 256 + d] +
                      hist[(k * 4 + 3) * 256 + d];
      coherent_store(&buf.table[((int64_t)k * 256 + d) * workers + wb], tot);
    }
    if (!sweeper_barrier(ctrl, ++gen, 0, &dummy, spin_limit, scratch)) return false;
    // ---- 2. per (segment, digit): exclusive prefix over the blocks, digit total
    for (int item = wb * 4 + wave; item < nseg * 256; item += workers * 4) {
      int* row = buf.table + (int64_t)item * workers;
      int carry = 0;
      constexpr int kChunks = (kRadixMaxWorkers + 63) / 64;  // all counts of the item are fetched together
      int vals[kChunks];
#pragma unroll
      for (int c = 0; c < kChunks; ++c) {
        const int b = c * 64 + lane;
        vals[c] = b < workers ? coherent_load(&row[b]) : 0;
      }
#pragma unroll
      for (int c = 0; c < kChunks; ++c) {
        const int b0 = c * 64;
        if (b0 >= workers) break;  // wave-uniform
        const int b = b0 + lane;
        const int v = vals[c];
        int incl = v;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
          const int up = __shfl_up(incl, off);
          if (lane >= off) incl += up;
        }
        if (b < workers) coherent_store(&row[b], carry + incl - v);
        carry += __shfl(incl, 63);
      }
      if (lane == 0) coherent_store(&buf.totals[item], carry);
    }
    if (!sweeper_barrier(ctrl, ++gen, 0, &dummy, spin_limit, scratch)) return false;
    // ---- 3. destinations and the stable move
    for (int k = 0; k < nseg; ++k) {
      const int d = threadIdx.x;
      const int tot = coherent_load(&buf.totals[k * 256 + d]);
      int incl = tot;
#pragma unroll
      for (int off = 1; off < 64; off <<= 1) {
        const int up = __shfl_up(incl, off);
        if (lane >= off) incl += up;
      }
      if (lane == 63) base[wave] = incl;
      __syncthreads();
      int first = incl - tot;
      for (int v = 0; v < wave; ++v) first += base[v];
      __syncthreads();
      // first destination of digit d for wave 0 of this block, then for waves 1..3
      int r = first + coherent_load(&buf.table[((int64_t)k * 256 + d) * workers + wb]);
      for (int v = 0; v < 4; ++v) {
        const int c = hist[(k * 4 + v) * 256 + d];
        hist[(k * 4 + v) * 256 + d] = r;
        r += c;
      }
    }
    __syncthreads();
    for (int k = 0; k < nseg; ++k) {
      int* h = hist + (k * 4 + wave) * 256;
      for (int b0 = w_begin; b0 < w_end; b0 += 64 * kRadixBatch) {
        unsigned long long batch[kRadixBatch];
#pragma unroll
        for (int u = 0; u < kRadixBatch; ++u) {
          const int e = b0 + 64 * u + lane;
          batch[u] = e >= w_end ? 0ull : (pass == 0 ? initial(k, e) : coherent_load(&in[(int64_t)k * buf.kstride + e]));
        }
#pragma unroll
        for (int u = 0; u < kRadixBatch; ++u) {
        const int e0 = b0 + 64 * u;
        if (e0 >= w_end) break;  // wave-uniform
        const int e = e0 + lane;
        const bool have = e < w_end;
        const unsigned long long p = batch[u];
        const int d = (int)((p >> (32 + shift)) & 255ull);
        // lanes of this group that hold the same digit
        uint64_t same = __builtin_amdgcn_ballot_w64(have);
#pragma unroll
        for (int bit = 0; bit < 8; ++bit) {
          const uint64_t b = __builtin_amdgcn_ballot_w64((d >> bit) & 1);
          same &= ((d >> bit) & 1) ? b : ~b;
        }
        const int leader = __ffsll((unsigned long long)same) - 1;
        const int rank = __popcll(same & ((1ull << lane) - 1ull));
        int start = 0;
        if (have && lane == leader) {
          start = h[d];
          h[d] = start + __popcll(same);
        }
        start = __shfl(start, leader < 0 ? 0 : leader);
        if (have) coherent_store(&out[(int64_t)k * buf.kstride + start + rank], p);
        }
      }
    }
    if (!sweeper_barrier(ctrl, ++gen, 0, &dummy, spin_limit, scratch)) return false;
  }
  return true;
}

// Block 0 of a radix kernel: the barrier master for `generations` barriers (12 per sort).
__device__ inline void radix_master(Ctrl* ctrl, unsigned gen0, unsigned generations, unsigned spin_limit, int* scratch) {
  int dummy = 0;
  for (unsigned g = 1; g <= generations; ++g)
    if (!master_barrier(ctrl, gen0 + g, 0, &dummy, spin_limit, scratch)) return;
}

// Barrier generations of the sorts start above every generation the peel can reach, and every run of
// a radix kernel takes a fresh range (the epoch counter lives in the control block).
__device__ inline unsigned radix_generation_base(const Ctrl* ctrl) { return 0x80000000u + 16u * (unsigned)ctrl->radix_epoch; }

// One step of the reference's lexsort (src/evox/utils/jit_fix_operator.py:246-250): positions ordered by
// key[prev[e]] ascending (NaN last, signed zeros tied), ties by position e, mapped back through prev --
//     sorted_key = key.gather(dim, sorted_indices); step = argsort(sorted_key, stable=True);
//     sorted_indices = sorted_indices.gather(dim, step)
// -- and the first step with prev == nullptr (the identity).  The caller chains one launch per key.
// kind 0: float32 keys, 1: int32 keys, 2: uint32 keys; `stride` in elements.
enum KeyKind { kKeyFloat32 = 0, kKeyInt32 = 1, kKeyUint32 = 2 };

__global__ __launch_bounds__(kRadixThreads) void argsort_step_kernel(const void* __restrict__ key, int kind, int64_t stride,
                                                                     int n, const int* __restrict__ prev,
                                                                     Ctrl* __restrict__ ctrl, RadixBuffers buf,
                                                                     int* __restrict__ order_out, unsigned spin_limit) {
  extern __shared__ int radix_lds[];
  __shared__ int base[256];
  __shared__ int scratch[kRadixThreads];
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
  auto initial = [&](int, int e) {
    const int idx = prev ? prev[e] : e;
    uint32_t k;
    if (kind == kKeyFloat32)
      k = ordered_key(static_cast<const float*>(key)[(int64_t)idx * stride]);
    else if (kind == kKeyInt32)
      k = static_cast<const uint32_t*>(key)[(int64_t)idx * stride] ^ 0x80000000u;
    else
      k = static_cast<const uint32_t*>(key)[(int64_t)idx * stride];
    return ((unsigned long long)k << 32) | (unsigned)idx;
  };
  if (!radix_sort_segments(buf, 1, n, initial, ctrl, gen0, spin_limit, radix_lds, base, scratch)) return;
  for (int p = wb * blockDim.x + threadIdx.x; p < n; p += workers * blockDim.x)
    order_out[p] = (int)(unsigned)(coherent_load(&buf.pairs[0][p]) & 0xFFFFFFFFull);
}

// The same step for at most kSmallArgsortRows positions in one launch, with no dependence between
// workgroups: every workgroup builds all composites (key << 14 | position, below 2^46, held as doubles:
// exact, and compared at the rate of 32-bit values) in LDS and places its own sixteen positions by counting
// the smaller composites, the count of a position split over 64 parts (the four quarters of a wave's lanes
// times the sixteen waves).  Same ordering as the radix sort: key ascending, ties by position.
constexpr int kSmallArgsortRows = 8192;  // measured per step: 30 us up to 8192 positions (radix sort: 90), 75 us at 16384
constexpr int kSmallArgsortThreads = 1024;
constexpr int kSmallArgsortGroup = 16;

__global__ __launch_bounds__(kSmallArgsortThreads) void small_argsort_kernel(const void* __restrict__ key, int kind, int64_t stride,
                                                                             int n, const int* __restrict__ prev,
                                                                             int* __restrict__ order_out) {
  extern __shared__ double argsort_comp[];  // n rounded up to a multiple of 128 entries, +inf past n
  __shared__ int share[16 * (64 / kSmallArgsortGroup)][kSmallArgsortGroup];
  const int npad = (n + 127) & ~127;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int e = threadIdx.x; e < npad; e += kSmallArgsortThreads) {
    double c = (double)INFINITY;
    if (e < n) {
      const int idx = prev ? prev[e] : e;
      uint32_t k;
      if (kind == kKeyFloat32)
        k = ordered_key(static_cast<const float*>(key)[(int64_t)idx * stride]);
      else if (kind == kKeyInt32)
        k = static_cast<const uint32_t*>(key)[(int64_t)idx * stride] ^ 0x80000000u;
      else
        k = static_cast<const uint32_t*>(key)[(int64_t)idx * stride];
      c = (double)(((uint64_t)k << 14) | (uint64_t)e);
    }
    argsort_comp[e] = c;
  }
  __syncthreads();
  constexpr int kParts = 16 * (64 / kSmallArgsortGroup);
  const int in_group = lane & (kSmallArgsortGroup - 1);
  const int split = wave * (64 / kSmallArgsortGroup) + lane / kSmallArgsortGroup;
  for (int e0 = blockIdx.x * kSmallArgsortGroup; e0 < npad; e0 += gridDim.x * kSmallArgsortGroup) {
    const int e = e0 + in_group;
    const double mine = argsort_comp[e];
    const int per = (((n + kParts - 1) / kParts) + 1) & ~1;
    const int b0 = split * per;
    const int b1 = min(b0 + per, (n + 1) & ~1);  // an odd n reads one entry of the padding: +inf
    int before = 0;
#pragma unroll 8
    for (int b = b0; b < b1; b += 2) {
      const double2 c = *reinterpret_cast<const double2*>(argsort_comp + b);
      before += (c.x < mine) + (c.y < mine);
    }
    share[split][in_group] = before;
    __syncthreads();
    if (wave == 0) {
      before = 0;
      const int q0 = (lane / kSmallArgsortGroup) * (kParts / (64 / kSmallArgsortGroup));
#pragma unroll
      for (int p = 0; p < kParts / (64 / kSmallArgsortGroup); ++p) before += share[q0 + p][in_group];
#pragma unroll
      for (int off = kSmallArgsortGroup; off < 64; off <<= 1) before += __shfl_xor(before, off);
      if (lane < kSmallArgsortGroup && e < n) order_out[before] = prev ? prev[e] : e;
    }
    __syncthreads();
  }
}

}  // namespace evx
