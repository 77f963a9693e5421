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
//   1. every block counts the digits of its chunks (LDS); the counts go to table[segment][digit][chunk];
//   2. for every (segment, digit) one wave turns the per-chunk counts into exclusive prefixes and
//      leaves the digit total;
//   3. every block scans the 256 digit totals of its chunk's segment, derives the destination of the chunk's
//      pairs of each digit, and moves the pairs tile by tile through LDS: inside a group of 64 pairs the rank
//      among equal digits comes from eight ballots, the waves and groups follow one another, so every pass is
//      stable.
// Pairs travel between blocks through relaxed agent-scope loads and stores (no cache-wide fences).
// The sizes are read from device memory, so the host launches this unconditionally; when the front is
// small the kernel returns at once.
#pragma once

#include "common.hpp"
#include "peel.hpp"

namespace evx {

constexpr int kRadixMinCandidates = 8192;
constexpr int kRadixThreads = 256;
constexpr int kRadixBatch = 4;  // pairs per lane fetched together when the digits are counted
constexpr int kRadixMaxWorkers = 510;  // working blocks of a radix kernel, at most (columns of the digit table)

struct RadixBuffers {
  unsigned long long* pairs[2];  // [segments][kstride] each: (key << 32) | candidate index
  int* table;                    // [segments][256][chunks], chunks <= kRadixMaxWorkers
  int* totals;                   // [segments][256]
  int kstride;
};

// Sorts `nseg` segments of nv pairs; pair e of segment k is initial(k, e) (candidate order), the
// result is left in buf.pairs[0] (four passes: initial -> pairs[1] -> pairs[0] -> pairs[1] -> pairs[0]; `passes` = 2
// where every key is below 65536: the same in all blocks, and the master runs three barriers per pass).
// Must be called by every thread of every block with blockIdx.x >= kFirstSweeper; block 0 must run
// radix_master().  `lds` = kRadixLdsBytes of LDS; `base` = LDS, 256 ints; `scratch` as for the barrier.
//
// A segment is cut into chunks (as many pairs as gives every working block about one chunk, a multiple of 256), and
// a block takes whole chunks: all pairs that it moves in a pass belong to one segment and lie side by side.  It
// stages them in LDS, a tile of kRadixTile at a time, in the order of their destinations, so that the pairs of one
// digit leave as one run of neighbouring addresses instead of one 8-byte store each.
constexpr int kRadixTile = 4096;
constexpr size_t kRadixLdsBytes = sizeof(int) * 6 * 256 + sizeof(unsigned long long) * kRadixTile;

template <class Initial>
__device__ inline bool radix_sort_segments(const RadixBuffers& buf, int nseg, int nv, Initial initial, Ctrl* ctrl,
                                           unsigned gen0, unsigned spin_limit, int* lds, int* base, int* scratch,
                                           int passes = 4) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int tid = threadIdx.x;  // blockDim.x == 256
  const int workers = gridDim.x - kFirstSweeper;
  const int wb = (int)blockIdx.x - kFirstSweeper;
  int64_t per = ((int64_t)nv * nseg + workers - 1) / workers;
  const int64_t least = ((int64_t)nv + kRadixMaxWorkers - 1) / kRadixMaxWorkers;  // the digit table has kRadixMaxWorkers columns
  if (per < least) per = least;
  const int chunk = (int)round_up(per < 256 ? 256 : per, 256);
  const int chunks = (nv + chunk - 1) / chunk;
  const int items = nseg * chunks;
  int* const hw = lds;               // [4][256]: digit counts of a tile per wave, then the waves' cursors
  int* const lstart = lds + 4 * 256;  // [256]: first staged position of every digit of the tile
  int* const gstart = lds + 5 * 256;  // [256]: destination of the next pair of every digit of the chunk
  unsigned long long* const stage = reinterpret_cast<unsigned long long*>(lds + 6 * 256);  // [kRadixTile]
  // exclusive prefix over the 256 threads of the block (two barriers)
  auto exclusive256 = [&](int v) {
    int incl = v;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const int up = __shfl_up(incl, off);
      if (lane >= off) incl += up;
    }
    if (lane == 63) base[wave] = incl;
    __syncthreads();
    int r = incl - v;
    for (int x = 0; x < wave; ++x) r += base[x];
    __syncthreads();
    return r;
  };
  unsigned gen = gen0;
  int dummy = 0;
  for (int pass = 0; pass < passes; ++pass) {
    const int shift = 8 * pass;
    // (chosen, not indexed: an array indexed at run time lives in scratch memory, which every lane of every kernel that
    // holds a RadixBuffers then writes when it starts -- 10 MB per launch of the 1024-thread ordering kernel)
    const unsigned long long* __restrict__ in = (pass & 1) ? buf.pairs[1] : buf.pairs[0];
    unsigned long long* __restrict__ out = (pass & 1) ? buf.pairs[0] : buf.pairs[1];
    auto fetch = [&](int k, int e) { return pass == 0 ? initial(k, e) : coherent_load(&in[(int64_t)k * buf.kstride + e]); };
    // ---- 1. digit counts of every chunk (kRadixBatch pairs per lane are fetched before any is used: the coherent
    // loads of a wave are then in flight together instead of costing a memory round trip each)
    for (int item = wb; item < items; item += workers) {
      const int k = item / chunks, c = item - k * chunks;
      const int begin = c * chunk, end = min(nv, begin + chunk);
      hw[tid] = 0;
      __syncthreads();
      for (int e0 = begin + tid; e0 < end; e0 += 256 * kRadixBatch) {
        unsigned long long p[kRadixBatch];
#pragma unroll
        for (int u = 0; u < kRadixBatch; ++u) p[u] = e0 + 256 * u < end ? fetch(k, e0 + 256 * u) : 0ull;
#pragma unroll
        for (int u = 0; u < kRadixBatch; ++u)
          if (e0 + 256 * u < end) atomicAdd(&hw[(int)((p[u] >> (32 + shift)) & 255ull)], 1);
      }
      __syncthreads();
      coherent_store(&buf.table[((int64_t)k * 256 + tid) * chunks + c], hw[tid]);
    }
    if (!sweeper_barrier(ctrl, ++gen, 0, &dummy, spin_limit, scratch)) return false;
    // ---- 2. per (segment, digit): exclusive prefix over the chunks, digit total
    for (int item = wb * 4 + wave; item < nseg * 256; item += workers * 4) {
      int* row = buf.table + (int64_t)item * chunks;
      int carry = 0;
      constexpr int kChunks = (kRadixMaxWorkers + 63) / 64;  // all counts of the item are fetched together
      int vals[kChunks];
#pragma unroll
      for (int q = 0; q < kChunks; ++q) {
        const int b = q * 64 + lane;
        vals[q] = b < chunks ? coherent_load(&row[b]) : 0;
      }
#pragma unroll
      for (int q = 0; q < kChunks; ++q) {
        const int b0 = q * 64;
        if (b0 >= chunks) break;  // wave-uniform
        const int b = b0 + lane;
        const int v = vals[q];
        int incl = v;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
          const int up = __shfl_up(incl, off);
          if (lane >= off) incl += up;
        }
        if (b < chunks) coherent_store(&row[b], carry + incl - v);
        carry += __shfl(incl, 63);
      }
      if (lane == 0) coherent_store(&buf.totals[item], carry);
    }
    if (!sweeper_barrier(ctrl, ++gen, 0, &dummy, spin_limit, scratch)) return false;
    // ---- 3. the stable move, chunk by chunk and tile by tile
    for (int item = wb; item < items; item += workers) {
      const int k = item / chunks, c = item - k * chunks;
      const int begin = c * chunk, end = min(nv, begin + chunk);
      {  // destination of the chunk's first pair of every digit: the smaller digits of the segment, then the earlier chunks
        const int total = coherent_load(&buf.totals[k * 256 + tid]);
        const int before = coherent_load(&buf.table[((int64_t)k * 256 + tid) * chunks + c]);
        gstart[tid] = exclusive256(total) + before;
      }
      for (int t0 = begin; t0 < end; t0 += kRadixTile) {
        const int count = min(end - t0, kRadixTile);
        const int sub = ((count + 255) / 256) * 64;  // a wave takes a quarter of the tile, whole groups of 64 pairs
        const int w_begin = min(count, wave * sub), w_end = min(count, w_begin + sub);
        constexpr int kGroups = kRadixTile / 4 / 64;
        unsigned long long pr[kGroups];
#pragma unroll
        for (int g = 0; g < kGroups; ++g) {
          const int e = w_begin + g * 64 + lane;
          pr[g] = e < w_end ? fetch(k, t0 + e) : 0ull;
        }
#pragma unroll
        for (int x = 0; x < 4; ++x) hw[x * 256 + tid] = 0;
        __syncthreads();
#pragma unroll
        for (int g = 0; g < kGroups; ++g)
          if (w_begin + g * 64 + lane < w_end) atomicAdd(&hw[wave * 256 + (int)((pr[g] >> (32 + shift)) & 255ull)], 1);
        __syncthreads();
        // staged position of the first pair of every digit, and from there the first pair of every wave
        const int c0 = hw[tid], c1 = hw[256 + tid], c2 = hw[512 + tid], c3 = hw[768 + tid];
        const int digit_total = c0 + c1 + c2 + c3;
        const int first = exclusive256(digit_total);
        lstart[tid] = first;
        hw[tid] = first;
        hw[256 + tid] = first + c0;
        hw[512 + tid] = first + c0 + c1;
        hw[768 + tid] = first + c0 + c1 + c2;
        __syncthreads();
        int* const cursor = hw + wave * 256;
#pragma unroll
        for (int g = 0; g < kGroups; ++g) {
          if (w_begin + g * 64 >= w_end) break;  // wave-uniform
          const bool have = w_begin + g * 64 + lane < w_end;
          const unsigned long long p = pr[g];
          const int d = (int)((p >> (32 + shift)) & 255ull);
          // lanes of this group that hold the same digit: the rank among them keeps the pass stable
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
            start = cursor[d];
            cursor[d] = start + __popcll(same);
          }
          start = __shfl(start, leader < 0 ? 0 : leader);
          if (have) stage[start + rank] = p;
        }
        __syncthreads();
        for (int t = tid; t < count; t += 256) {
          const unsigned long long p = stage[t];
          const int d = (int)((p >> (32 + shift)) & 255ull);
          coherent_store(&out[(int64_t)k * buf.kstride + gstart[d] + (t - lstart[d])], p);
        }
        __syncthreads();
        gstart[tid] += digit_total;  // read again after the barriers of the next tile, or not at all
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
// key_cap (device memory, or null): int32 keys that are not negative are sorted as min(key, *key_cap) -- two passes
// instead of four where the cap is below 65536 (the ranks of a population, whose number of fronts an earlier kernel
// has left there; rows without a rank stand behind all others either way).
enum KeyKind { kKeyFloat32 = 0, kKeyInt32 = 1, kKeyUint32 = 2 };

__global__ __launch_bounds__(kRadixThreads) void argsort_step_kernel(const void* __restrict__ key, int kind, int64_t stride,
                                                                     int n, const int* __restrict__ prev,
                                                                     Ctrl* __restrict__ ctrl, RadixBuffers buf,
                                                                     int* __restrict__ order_out, unsigned spin_limit,
                                                                     const int* __restrict__ key_cap) {
  extern __shared__ int radix_lds[];
  __shared__ int base[256];
  __shared__ int scratch[kRadixThreads];
  if (coherent_load(&ctrl->err) != 0) return;
  const unsigned gen0 = radix_generation_base(ctrl);
  const bool capped = key_cap != nullptr && kind == kKeyInt32;
  const uint32_t cap = capped ? (uint32_t)*key_cap : 0xFFFFFFFFu;
  const int passes = capped && cap < 65536u ? 2 : 4;
  if (blockIdx.x == 0) {
    radix_master(ctrl, gen0, 3 * passes, spin_limit, scratch);
    if (threadIdx.x == 0) ctrl->radix_epoch += 1;  // nobody reads it again in this kernel
    return;
  }
  if (blockIdx.x < kFirstSweeper) return;
  const int workers = gridDim.x - kFirstSweeper;
  const int wb = (int)blockIdx.x - kFirstSweeper;
  auto initial = [&](int, int e) {
    int idx = prev ? prev[e] : e;
    if (idx < 0) {  // the order of a step whose wait ran out (-1 everywhere): this step fails too, and reads nothing through it
      coherent_store(&ctrl->err, kErrBarrierTimeout);
      idx = 0;
    }
    uint32_t k;
    if (kind == kKeyFloat32)
      k = ordered_key(static_cast<const float*>(key)[(int64_t)idx * stride]);
    else if (capped)
      k = min(static_cast<const uint32_t*>(key)[(int64_t)idx * stride], cap);
    else if (kind == kKeyInt32)
      k = static_cast<const uint32_t*>(key)[(int64_t)idx * stride] ^ 0x80000000u;
    else
      k = static_cast<const uint32_t*>(key)[(int64_t)idx * stride];
    return ((unsigned long long)k << 32) | (unsigned)idx;
  };
  if (!radix_sort_segments(buf, 1, n, initial, ctrl, gen0, spin_limit, radix_lds, base, scratch, passes)) return;
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

// (blockIdx.y: one of several such steps in the launch, their keys key_step bytes and their orders order_step bytes apart)
__global__ __launch_bounds__(kSmallArgsortThreads) void small_argsort_kernel(const void* __restrict__ key, int kind, int64_t stride,
                                                                             int n, const int* __restrict__ prev,
                                                                             int* __restrict__ order_out, int64_t key_step = 0,
                                                                             int64_t order_step = 0) {
  extern __shared__ double argsort_comp[];  // n rounded up to a multiple of 128 entries, +inf past n
  key = static_cast<const char*>(key) + (int64_t)blockIdx.y * key_step;
  order_out = reinterpret_cast<int*>(reinterpret_cast<char*>(order_out) + (int64_t)blockIdx.y * order_step);
  if (prev != nullptr) prev = reinterpret_cast<const int*>(reinterpret_cast<const char*>(prev) + (int64_t)blockIdx.y * order_step);
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

// The same step for kSmallArgsortRows < n <= kMidArgsortRows positions, still in one launch with no dependence
// between workgroups (the radix sort needs three launches and twelve grid barriers: 70 us at 20 000 positions, more
// than torch's own sort).  Every workgroup reads all keys into LDS (32-bit order-preserving images) and works on
// composites (image << 15 | position: distinct, below 2^47); it produces a run of `slots_per_block` slots of the
// result: the histogram of all composites over 4096 (or 2048) buckets (LDS atomics), its scan, the buckets that
// hold the wanted slots, their composites collected into a list, every member of the list placed by counting the
// members below it (sixteen lanes per member).  Keys with few distinct values are the usual case here (ranks, a
// distance that is -inf for most rows): the buckets cut the composites, so a key held by thousands of positions is
// spread over many buckets by its position bits.  A group of buckets with more than kMidArgsortList composites is
// not collected: the workgroup takes the bucket of its next slot alone, and if that is too large as well (a wide
// range of keys with a crowd on one value) it builds the histogram of that bucket's range, which is narrower by the
// bucket count each time, down to single composites.  The code is loops, not unrolled passes: a launch starts with
// a cold instruction cache.
constexpr int kMidArgsortRows = 32768;  // keys of 4 bytes in LDS (128 KB) beside the tables: a merged population of 2 x 16384
constexpr int kMidArgsortThreads = 1024;
// Up to kMidArgsortWideRows keys the tables are 4096 buckets and a list of 2048 (48 KB); above, 2048 buckets and a list
// of 1536 (28 KB), so that 32768 keys still fit beside them (20 000 keys: 15 us slower with the small tables).
constexpr int kMidArgsortWideRows = 24576;
constexpr int kMidArgsortIndexBits = 15;

// Exclusive scan, in place, of the BUCKETS counts in `hist` by the whole workgroup; returns their sum.
template <int BUCKETS>
__device__ inline int mid_argsort_scan(int* hist, int* wave_tot) {
  constexpr int kPer = BUCKETS / kMidArgsortThreads;  // consecutive buckets per thread
  static_assert(kPer == 2 || kPer == 4, "two or four buckets per thread");
  constexpr int kWaves = kMidArgsortThreads / 64;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  int c[kPer];
  if constexpr (kPer == 4) {
    const int4 v = *reinterpret_cast<const int4*>(hist + tid * kPer);
    c[0] = v.x; c[1] = v.y; c[2] = v.z; c[3] = v.w;
  } else {
    const int2 v = *reinterpret_cast<const int2*>(hist + tid * kPer);
    c[0] = v.x; c[1] = v.y;
  }
  int mine = 0;
#pragma unroll
  for (int u = 0; u < kPer; ++u) mine += c[u];
  int incl = mine;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const int up = __shfl_up(incl, off);
    if (lane >= off) incl += up;
  }
  if (lane == 63) wave_tot[wave] = incl;
  __syncthreads();
  int run = incl - mine, total = 0;
#pragma unroll
  for (int w = 0; w < kWaves; ++w) {
    if (w < wave) run += wave_tot[w];
    total += wave_tot[w];
  }
#pragma unroll
  for (int u = 0; u < kPer; ++u) {
    hist[tid * kPer + u] = run;
    run += c[u];
  }
  __syncthreads();
  return total;
}

// The tables of a workgroup that sorts in LDS, carved from `bytes` = mid_sort_lds_bytes(n) of it.
struct MidSortLds {
  int* top_hist;             // [buckets] first-level starts, kept
  int* sub_hist;             // [buckets] starts of the level below, rebuilt
  unsigned long long* list;  // [list entries]
  uint32_t* red;             // [2][waves]
  int* wave_tot;             // [waves]
  int* found;                // [5] bucket of the first wanted slot, its start and end; bucket of the last wanted slot, its end
  int* list_count;
  uint32_t* keys;            // [n] order-preserving images of the keys, in the order of the positions
};
__host__ __device__ inline size_t mid_sort_table_bytes(int n) {
  const int buckets = n <= kMidArgsortWideRows ? 4096 : 2048, list = n <= kMidArgsortWideRows ? 2048 : 1536;
  return 2 * sizeof(int) * (size_t)buckets + sizeof(unsigned long long) * (size_t)list + 256;
}
__host__ __device__ inline size_t mid_sort_lds_bytes(int n) { return mid_sort_table_bytes(n) + sizeof(uint32_t) * (size_t)n; }
template <int BUCKETS, int LIST>
__device__ inline MidSortLds mid_sort_lds(void* lds) {  // (16-byte aligned)
  constexpr int kWaves = kMidArgsortThreads / 64;
  MidSortLds t;
  t.top_hist = static_cast<int*>(lds);
  t.sub_hist = t.top_hist + BUCKETS;
  t.list = reinterpret_cast<unsigned long long*>(t.sub_hist + BUCKETS);
  t.red = reinterpret_cast<uint32_t*>(t.list + LIST);
  t.wave_tot = reinterpret_cast<int*>(t.red + 2 * kWaves);
  t.found = t.wave_tot + kWaves;
  t.list_count = t.found + 5;
  t.keys = reinterpret_cast<uint32_t*>(reinterpret_cast<char*>(lds) + 2 * sizeof(int) * BUCKETS + sizeof(unsigned long long) * LIST + 256);
  return t;
}

// Slots s0 .. s1-1 of the stable ascending order of n <= kMidArgsortRows 32-bit keys, by one workgroup of
// kMidArgsortThreads threads that holds all keys in LDS and waits for no other workgroup: key_of(e) = the key of
// position e (read once), emit(slot, e) = position e belongs in `slot`.  The keys go into BUCKETS buckets
// by value; the buckets that hold the wanted slots are collected (a bucket too large for the list is cut into buckets
// of its own range first) and their members placed by counting.  Every thread of the workgroup calls it.
template <int BUCKETS, int LIST, int TRACE, class KeyOf, class Emit>
__device__ inline void mid_argsort_slice_sized(void* lds, int n, int s0, int s1_wanted, KeyOf key_of, Emit emit) {
  constexpr int kMidArgsortBuckets = BUCKETS, kMidArgsortList = LIST;
  const MidSortLds T = mid_sort_lds<BUCKETS, LIST>(lds);
  uint32_t* const mid_keys = T.keys;
  int* const top_hist = T.top_hist;
  int* const sub_hist = T.sub_hist;
  unsigned long long* const list = T.list;
  int* const wave_tot = T.wave_tot;
  int* const found = T.found;
  constexpr int kWaves = kMidArgsortThreads / 64;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  constexpr unsigned long long kIndexMask = (1ull << kMidArgsortIndexBits) - 1ull;
  uint32_t kmin = 0xFFFFFFFFu, kmax = 0u;
#pragma unroll 4
  for (int e = tid; e < n; e += kMidArgsortThreads) {
    const uint32_t k = key_of(e);
    mid_keys[e] = k;
    kmin = k < kmin ? k : kmin;
    kmax = k > kmax ? k : kmax;
  }
  EVX_TRACE(TRACE, 0);
  for (int b = tid; b < kMidArgsortBuckets; b += kMidArgsortThreads) top_hist[b] = 0;
  if (tid == 0) *T.list_count = 0;
  if (tid < 5) found[tid] = 0;
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const uint32_t a = __shfl_xor(kmin, off), b = __shfl_xor(kmax, off);
    kmin = a < kmin ? a : kmin;
    kmax = b > kmax ? b : kmax;
  }
  if (lane == 0) {
    T.red[wave] = kmin;
    T.red[kWaves + wave] = kmax;
  }
  __syncthreads();
#pragma unroll
  for (int w = 0; w < kWaves; ++w) {
    kmin = T.red[w] < kmin ? T.red[w] : kmin;
    kmax = T.red[kWaves + w] > kmax ? T.red[kWaves + w] : kmax;
  }
  auto composite = [&](int e) { return ((unsigned long long)mid_keys[e] << kMidArgsortIndexBits) | (unsigned long long)e; };
  auto shift_for = [](unsigned long long span) {
    int shift = 0;
    while (shift < 63 && (span >> shift) >= (unsigned long long)kMidArgsortBuckets) ++shift;
    return shift;
  };
  const unsigned long long top_lo = (unsigned long long)kmin << kMidArgsortIndexBits;
  const unsigned long long top_hi = ((unsigned long long)kmax << kMidArgsortIndexBits) | kIndexMask;
  const int top_shift = shift_for(top_hi - top_lo);
  for (int e = tid; e < n; e += kMidArgsortThreads) atomicAdd(&top_hist[(int)((composite(e) - top_lo) >> top_shift)], 1);
  __syncthreads();
  mid_argsort_scan<BUCKETS>(top_hist, wave_tot);  // (the total is n)
  EVX_TRACE(TRACE, 1);
  const int s1 = min(n, s1_wanted);
  // level state: the same in every thread
  unsigned long long lo = top_lo, hi = top_hi;  // the composites of the level: lo .. hi
  int shift = top_shift, base = 0, total = n;
  bool at_top = true;
  int x = s0;
  // (every round either places slots or narrows the range; the count is a guard against a loop that does neither)
  for (int rounds = 0; x < s1 && rounds < 8 * kMidArgsortList; ++rounds) {
    const int* hist = at_top ? top_hist : sub_hist;
    {
      // the buckets that hold slot x and the last wanted slot of this level
      const int q0 = x - base, q1 = min(s1 - 1 - base, total - 1);
      constexpr int kPer = kMidArgsortBuckets / kMidArgsortThreads;
#pragma unroll
      for (int u = 0; u < kPer; ++u) {
        const int b = u * kMidArgsortThreads + tid;  // (neighbouring lanes read neighbouring words)
        const int st = hist[b], en = b + 1 < kMidArgsortBuckets ? hist[b + 1] : total;
        if (st <= q0 && q0 < en) {
          found[0] = b;
          found[1] = st;
          found[2] = en;
        }
        if (st <= q1 && q1 < en) {
          found[3] = b;
          found[4] = en;
        }
      }
    }
    __syncthreads();
    const int b0 = found[0], b0_start = found[1], b0_end = found[2];
    int b1 = found[3], b1_end = found[4];
    // Placing the members of the collected buckets costs their number squared: where the keys crowd into a few buckets
    // (crowding distances do), a bucket many times larger than the run of slots that is wanted from it is cut up first.
    const int most = min(kMidArgsortList, max(512, 4 * (s1 - x)));
    if (b1_end - b0_start > most) {
      if (b0_end - b0_start > most) {
        // that bucket alone is too large: the histogram of its range
        base += b0_start;
        total = b0_end - b0_start;
        lo += (unsigned long long)b0 << shift;
        const unsigned long long span = (1ull << shift) - 1ull < hi - lo ? (1ull << shift) - 1ull : hi - lo;
        hi = lo + span;
        shift = shift_for(span);
        at_top = false;
        for (int b = tid; b < kMidArgsortBuckets; b += kMidArgsortThreads) sub_hist[b] = 0;
        __syncthreads();
        for (int e0 = 0; e0 < n; e0 += kMidArgsortThreads) {
          const int e = e0 + tid;
          const unsigned long long c = e < n ? composite(e) : 0ull;
          const bool in = e < n && c >= lo && c - lo <= span;
          const int b = in ? (int)((c - lo) >> shift) : -1;
          // (thousands of equal keys -- what makes a bucket too large in the first place -- fall into one bucket of
          // this level too, and additions to one LDS word are carried out one after the other: where all lanes of the
          // wave that have a key in the range have the same bucket, one of them adds for all)
          const uint64_t ins = __builtin_amdgcn_ballot_w64(in);
          if (ins != 0ull) {
            const int lead = __ffsll((unsigned long long)ins) - 1;
            const int b_lead = __builtin_amdgcn_readlane(b, lead);
            if (__builtin_amdgcn_ballot_w64(in && b == b_lead) == ins) {
              if (lane == lead) atomicAdd(&sub_hist[b_lead], __popcll(ins));
            } else if (in) {
              atomicAdd(&sub_hist[b], 1);
            }
          }
        }
        __syncthreads();
        mid_argsort_scan<BUCKETS>(sub_hist, wave_tot);
        continue;
      }
      // as many buckets from b0 on as the list takes (not b0 alone: where the run of wanted slots ends in a bucket of
      // thousands of equal keys, every round would place one small bucket): the last bucket that ends in time
      __syncthreads();  // (everybody has read found[])
      constexpr int kPer = kMidArgsortBuckets / kMidArgsortThreads;
#pragma unroll
      for (int u = 0; u < kPer; ++u) {
        const int b = u * kMidArgsortThreads + tid;
        const int en = b + 1 < kMidArgsortBuckets ? hist[b + 1] : total;
        const int en_next = b + 2 < kMidArgsortBuckets ? hist[b + 2] : total;
        if (b >= b0 && en - b0_start <= most && (en_next - b0_start > most || b + 1 >= kMidArgsortBuckets)) {
          found[3] = b;
          found[4] = en;
        }
      }
      __syncthreads();
      b1 = found[3];
      b1_end = found[4];
    }
    {
      const unsigned long long first = lo + ((unsigned long long)b0 << shift);
      const unsigned long long width = ((unsigned long long)(b1 - b0 + 1) << shift) - 1ull;  // composites first .. first + width
      // (one addition to the list's counter per wave, not per member: thousands of them to one LDS word take longer
      // than everything else in a round)
      for (int e0 = 0; e0 < n; e0 += kMidArgsortThreads) {
        const int e = e0 + tid;
        const unsigned long long c = e < n ? composite(e) : 0ull;
        const bool take = e < n && c >= first && c - first <= width && c <= hi;
        const unsigned long long takers = __builtin_amdgcn_ballot_w64(take);
        if (takers != 0ull) {
          int at = 0;
          if (lane == 0) at = atomicAdd(T.list_count, __popcll(takers));
          at = __shfl(at, 0);
          if (take) list[at + __popcll(takers & ((1ull << lane) - 1ull))] = c;
        }
      }
    }
    __syncthreads();
    EVX_TRACE(TRACE, 2);
    const int members = *T.list_count;  // = b1_end - b0_start
    // sixteen lanes per member: each counts over a sixteenth of the list, the shares are added inside the DPP row
    for (int p0 = 0; p0 < members; p0 += kMidArgsortThreads / 16) {
      const int p = p0 + (tid >> 4), sub = tid & 15;
      const unsigned long long c = p < members ? list[p] : 0ull;
      int before = 0;
#pragma unroll 4
      for (int q = sub; q < members; q += 16) before += list[q] < c;
      before = group16_sum(before);
      const int slot = base + b0_start + before;
      if (sub == 0 && p < members && slot >= x && slot < s1) emit(slot, (int)(c & kIndexMask));
    }
    x = base + b1_end;
    __syncthreads();  // the list and found[] are rewritten
    if (tid == 0) *T.list_count = 0;
    // back to the first level for the slots that are left, unless the next of them lies in the range of this level too
    // (its histogram is still there: a run of slots inside thousands of equal keys is cut up once, not once per round)
    if (!at_top && !(x < base + total)) {
      lo = top_lo;
      hi = top_hi;
      shift = top_shift;
      base = 0;
      total = n;
      at_top = true;
    }
  }
  __syncthreads();
  EVX_TRACE(TRACE, 3);
}

// WIDE: the large tables (at most kMidArgsortWideRows keys).  `lds` = mid_sort_lds_bytes(most keys the launch may
// meet) bytes, 16-byte aligned: the host picks WIDE by that number, so that a kernel holds one size of the code.
template <bool WIDE, int TRACE = 51, class KeyOf, class Emit>
__device__ inline void mid_argsort_slice(void* lds, int n, int s0, int s1_wanted, KeyOf key_of, Emit emit) {
  if constexpr (WIDE)
    mid_argsort_slice_sized<4096, 2048, TRACE>(lds, n, s0, s1_wanted, key_of, emit);
  else
    mid_argsort_slice_sized<2048, 1536, TRACE>(lds, n, s0, s1_wanted, key_of, emit);
}

// One step of a lexsort of n <= kMidArgsortRows positions: a workgroup per `slots_per_block` slots of the order.
// Dynamic LDS: mid_sort_lds_bytes(n).
template <bool WIDE>
__global__ __launch_bounds__(kMidArgsortThreads) void mid_argsort_kernel(const void* __restrict__ key, int kind, int64_t stride, int n,
                                                                         const int* __restrict__ prev, int slots_per_block,
                                                                         int* __restrict__ order_out, int64_t key_step = 0,
                                                                         int64_t order_step = 0) {
  extern __shared__ __attribute__((aligned(16))) unsigned char mid_lds[];
  // (blockIdx.y: one of several such steps in the launch, their keys key_step bytes and their orders order_step bytes apart)
  key = static_cast<const char*>(key) + (int64_t)blockIdx.y * key_step;
  order_out = reinterpret_cast<int*>(reinterpret_cast<char*>(order_out) + (int64_t)blockIdx.y * order_step);
  if (prev != nullptr) prev = reinterpret_cast<const int*>(reinterpret_cast<const char*>(prev) + (int64_t)blockIdx.y * order_step);
  auto key_of = [&](int e) -> uint32_t {
    const int idx = prev ? prev[e] : e;
    if (kind == kKeyFloat32) return ordered_key(static_cast<const float*>(key)[(int64_t)idx * stride]);
    if (kind == kKeyInt32) return static_cast<const uint32_t*>(key)[(int64_t)idx * stride] ^ 0x80000000u;
    return static_cast<const uint32_t*>(key)[(int64_t)idx * stride];
  };
  const int s0 = (int)blockIdx.x * slots_per_block;
  mid_argsort_slice<WIDE>(mid_lds, n, s0, s0 + slots_per_block, key_of, [&](int slot, int e) { order_out[slot] = prev ? prev[e] : e; });
}

// Many independent steps at once: `batch` sorts of n <= kSmallArgsortRows positions each, sort b reading
// key[b * batch_stride + idx * stride], prev[b * n + .] and writing order_out[b * n + .].  A workgroup of T
// threads takes `rows_per_block` sorts at a time (a power of two; T / rows_per_block threads each) with the
// composites of its sorts in LDS; a thread keeps up to R positions of one sort in registers and counts, in one
// pass over that sort's composites, how many of them precede each of its own.  Needs
// n <= R * T / rows_per_block.  LDS: rows_per_block * row_stride doubles, row_stride >= n (odd when several
// sorts share a workgroup, so that their reads fall into different banks).
template <int T, int R>
__global__ __launch_bounds__(T) void rows_argsort_kernel(const void* __restrict__ key, int kind, int64_t batch_stride, int64_t stride,
                                                         int64_t batch, int n, int rows_per_block, int row_stride,
                                                         const int* __restrict__ prev, int* __restrict__ order_out) {
  extern __shared__ double rows_comp[];
  const int group = T / rows_per_block;
  const int local_row = threadIdx.x / group;
  const int in_group = threadIdx.x - local_row * group;
  for (int64_t row0 = (int64_t)blockIdx.x * rows_per_block; row0 < batch; row0 += (int64_t)gridDim.x * rows_per_block) {
    const int64_t row = row0 + local_row;
    const bool live = row < batch;
    double* const comp = rows_comp + (size_t)local_row * row_stride;
    const int* const prev_row = prev ? prev + row * n : nullptr;
    if (live) {
      for (int e = in_group; e < n; e += group) {
        const int idx = prev_row ? prev_row[e] : e;
        const int64_t at = row * batch_stride + (int64_t)idx * stride;
        uint32_t k;
        if (kind == kKeyFloat32)
          k = ordered_key(static_cast<const float*>(key)[at]);
        else if (kind == kKeyInt32)
          k = static_cast<const uint32_t*>(key)[at] ^ 0x80000000u;
        else
          k = static_cast<const uint32_t*>(key)[at];
        comp[e] = (double)(((uint64_t)k << 14) | (uint64_t)e);
      }
    }
    __syncthreads();
    double mine[R];
    int before[R];
#pragma unroll
    for (int q = 0; q < R; ++q) {
      const int e = in_group + q * group;
      mine[q] = (live && e < n) ? comp[e] : 0.0;  // nothing precedes zero: idle positions count nothing
      before[q] = 0;
    }
    if (live) {
#pragma unroll 8
      for (int b = 0; b < n; ++b) {
        const double c = comp[b];
#pragma unroll
        for (int q = 0; q < R; ++q) before[q] += c < mine[q] ? 1 : 0;
      }
#pragma unroll
      for (int q = 0; q < R; ++q) {
        const int e = in_group + q * group;
        if (e < n) order_out[row * n + before[q]] = prev_row ? prev_row[e] : e;
      }
    }
    __syncthreads();
  }
}

// Longer sorts of a batch, one workgroup per sort: the composites (key << 14 | position, distinct, so any
// sorting network gives the stable order) go through a bitonic network in LDS, padded with +inf to npad, a
// power of two from 512 to kRowsArgsortMax.  A thread takes eight entries at a time into registers and runs up
// to three stages of the network on them before they go back, so a sort of 8192 makes 33 passes over LDS for
// its 91 stages: entries 8t .. 8t+7 are sorted outright first (the phases of length 2, 4 and 8), and the
// stages of a later phase are grouped by the index bits they pair, {2,1,0}, {5,4,3}, {8,7,6}, ..., the top
// group taking what is left.  Entry e lives at e ^ swizzle(e), which keeps the 32 lanes of a half wave on 32
// different banks in every full group.  O(n log^2 n) compare-exchanges per sort, where counting needs n^2
// comparisons.
constexpr int kRowsArgsortMax = 16384;  // positions per sort (14 bits of a composite), 128 KB of LDS
constexpr int kRowsBitonicMin = 512;    // smallest padded length (one wave, eight entries per lane)

__device__ inline int bitonic_slot(int e) { return e ^ ((e >> 5) & 7) ^ (((e >> 6) & 3) << 3); }

__device__ inline void compare_exchange(double& a, double& b) {
  const double lo = __builtin_fmin(a, b), hi = __builtin_fmax(a, b);
  a = lo;
  b = hi;
}

// The stages of phase k that pair entries differing in one of the S index bits low_log .. low_log + S - 1.
template <int S>
__device__ inline void bitonic_pass(double* comp, int npad, int k, int low_log) {
  constexpr int E = 1 << S;
  const int units = npad >> S;
  for (int u = threadIdx.x; u < units; u += blockDim.x) {
    const int base = ((u >> low_log) << (low_log + S)) | (u & ((1 << low_log) - 1));
    const int flip = (base & k) ? E - 1 : 0;  // a descending run is an ascending one read backwards
    double v[E];
#pragma unroll
    for (int c = 0; c < E; ++c) v[c] = comp[bitonic_slot(base + ((c ^ flip) << low_log))];
#pragma unroll
    for (int d = E >> 1; d > 0; d >>= 1)
#pragma unroll
      for (int c = 0; c < E; ++c)
        if ((c & d) == 0) compare_exchange(v[c], v[c | d]);
#pragma unroll
    for (int c = 0; c < E; ++c) comp[bitonic_slot(base + ((c ^ flip) << low_log))] = v[c];
  }
}

// Sorts comp[bitonic_slot(0 .. npad-1)] ascending in place: npad a power of two from kRowsBitonicMin on, the entries
// distinct or +inf.  Every thread of the workgroup calls it, after a barrier that follows the last write of an entry;
// it ends with a barrier.
__device__ inline void bitonic_sort_lds(double* comp, int npad) {
  // phases 2, 4 and 8: eight neighbours sorted in registers, every second run of eight descending
  for (int u = threadIdx.x; u < (npad >> 3); u += blockDim.x) {
    const int base = u << 3;
    const int flip = (base & 8) ? 7 : 0;
    double v[8];
#pragma unroll
    for (int c = 0; c < 8; ++c) v[c] = comp[bitonic_slot(base + (c ^ flip))];
    compare_exchange(v[0], v[1]); compare_exchange(v[3], v[2]); compare_exchange(v[4], v[5]); compare_exchange(v[7], v[6]);
    compare_exchange(v[0], v[2]); compare_exchange(v[1], v[3]); compare_exchange(v[6], v[4]); compare_exchange(v[7], v[5]);
    compare_exchange(v[0], v[1]); compare_exchange(v[2], v[3]); compare_exchange(v[5], v[4]); compare_exchange(v[7], v[6]);
#pragma unroll
    for (int d = 4; d > 0; d >>= 1)
#pragma unroll
      for (int c = 0; c < 8; ++c)
        if ((c & d) == 0) compare_exchange(v[c], v[c | d]);
#pragma unroll
    for (int c = 0; c < 8; ++c) comp[bitonic_slot(base + (c ^ flip))] = v[c];
  }
  __syncthreads();
  for (int k = 16, top = 3; k <= npad; k <<= 1, ++top) {  // top = the highest index bit that phase k pairs
    int low_log = (top / 3) * 3;
    const int first = top - low_log + 1;
    if (first == 1)
      bitonic_pass<1>(comp, npad, k, low_log);
    else if (first == 2)
      bitonic_pass<2>(comp, npad, k, low_log);
    else
      bitonic_pass<3>(comp, npad, k, low_log);
    __syncthreads();
    for (low_log -= 3; low_log >= 0; low_log -= 3) {
      bitonic_pass<3>(comp, npad, k, low_log);
      __syncthreads();
    }
  }
}

__global__ __launch_bounds__(1024) void rows_bitonic_argsort_kernel(const void* __restrict__ key, int kind, int64_t batch_stride,
                                                                    int64_t stride, int64_t batch, int n, int npad,
                                                                    const int* __restrict__ prev, int* __restrict__ order_out) {
  extern __shared__ double bitonic_comp[];
  double* const comp = bitonic_comp;
  for (int64_t row = blockIdx.x; row < batch; row += gridDim.x) {
    const int* const prev_row = prev ? prev + row * n : nullptr;
    for (int e = threadIdx.x; e < npad; e += blockDim.x) {
      double c = (double)INFINITY;
      if (e < n) {
        const int idx = prev_row ? prev_row[e] : e;
        const int64_t at = row * batch_stride + (int64_t)idx * stride;
        uint32_t k;
        if (kind == kKeyFloat32)
          k = ordered_key(static_cast<const float*>(key)[at]);
        else if (kind == kKeyInt32)
          k = static_cast<const uint32_t*>(key)[at] ^ 0x80000000u;
        else
          k = static_cast<const uint32_t*>(key)[at];
        c = (double)(((uint64_t)k << 14) | (uint64_t)e);
      }
      comp[bitonic_slot(e)] = c;
    }
    __syncthreads();
    bitonic_sort_lds(comp, npad);
    for (int e = threadIdx.x; e < n; e += blockDim.x) {
      const int pos = (int)((uint64_t)comp[bitonic_slot(e)] & 16383ull);
      order_out[row * n + e] = prev_row ? prev_row[pos] : pos;
    }
    __syncthreads();
  }
}

}  // namespace evx
