// Domination counts and front peeling over the dominated-by bit matrix.
//
// Reference semantics:
//   count[j] = sum_i A[i, j]                                   src/evox/operators/selection/non_dominate.py:188
//   front    = count == 0                                      non_dominate.py:192
//   repeat while the front is not empty (non_dominate.py:161-169):
//     rank[front] = level; count -= sum_{i in front} A[i, :]; count -= front (non_dominate.py:29-59)
//     level += 1; front = count == 0
//
// Row j of the matrix (slot space, see order.hpp) is the dominator set of j, so count[j] =
// popcount(row j) and a row enters the next front exactly when no unranked row dominates it any more.
// Two interchangeable passes implement that:
//   * the sweep pass keeps the counts: count[j] -= popcount(row j & front) for every unranked row;
//   * the witness pass keeps, per unranked row, one word of its row that still holds an unranked
//     dominator, and touches memory only when that word has none left.
// Because the matrix is strictly lower triangular, only words 0 .. j/64 of row j are ever read.
//
// The pass loop runs inside ONE persistent kernel: the sweeping blocks meet at a grid barrier after
// every pass and learn the size of the next front from the barrier itself, so the host never waits
// for a front.  A separate block lists every finished front in ascending original row index into
// `perm` (a stable ordering by rank, which is what the final selection needs for every rank better
// than the last one) off the critical path.
#pragma once

#include "common.hpp"

// Hooks for development builds; they compile to nothing in the library.
#ifndef EVX_TRACE
#define EVX_TRACE(level, slot)
#endif
#ifndef EVX_TRACE_POOL
#define EVX_TRACE_POOL(level, slot)
#endif
#ifndef EVX_RESCAN
#define EVX_RESCAN(level, rows, rounds)
#endif

namespace evx {

constexpr int kPeelThreads = 256;
// Words of a front bitmap in global memory are kFrontStride words apart (one per 128-byte line): the
// rows of a front are published by many waves at the same moment, and atomics that share a line
// serialise.
constexpr int kFrontStride = 16;

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also waits for every outstanding
// global load of the wave, which a pass of the persistent kernels has no reason to wait for.
__device__ inline void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// Clears the control block, the front sizes, the front bitmaps and the sort histogram (one region).
__global__ __launch_bounds__(256) void reset_state_kernel(uint32_t* __restrict__ words, int64_t n_words) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n_words; i += (int64_t)gridDim.x * blockDim.x)
    words[i] = 0u;
}

// dst[i] = src[i] (4-byte elements), or `poison` everywhere when a device-side wait of the call ran out: the last
// kernel of an entry point, so that a caller who never reads the status still cannot take a partial result for a
// result (ranks -1, distances NaN, orders -1).  src == nullptr only poisons.
__global__ __launch_bounds__(256) void copy_or_poison_kernel(const Ctrl* __restrict__ ctrl, const uint32_t* __restrict__ src,
                                                             uint32_t* __restrict__ dst, int64_t n, uint32_t poison,
                                                             int64_t ws_step) {
  // (several populations in one launch: their results lie n elements apart)
  to_population(ws_step, ctrl, src);
  dst += (int64_t)blockIdx.z * n;
  const bool failed = ctrl->err != 0;
  if (!failed && src == nullptr) return;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
    dst[i] = failed ? poison : src[i];
}

// Words of row j that can hold a dominator (slots below j), rounded up to a whole 16-byte pair.
__device__ inline int row_words(int j) { return ((j >> 6) + 2) & ~1; }

// ---------------------------------------------------------------- row scan

// Wave-cooperative scan of R bit rows at once (optionally ANDed with a bitmap in LDS).  Every lane
// takes pairs of words 128 apart; the loads of a U*128-word stretch of all R rows are issued before
// any of them is used, so a scan costs about one memory latency however many rows are scanned
// together.  Per row it returns the popcount, the highest non-empty word (-1 when the row is empty)
// and that word's unmasked value, identical in every lane.
struct RowScan {
  int total;
  int last_word;
  uint64_t last_bits;
};

// Wave-wide sum and maximum through DPP row shifts and row broadcasts (vector ALU, a few clocks per
// step) instead of six dependent steps through the LDS permute unit.  The result is the same in all lanes.
__device__ inline int wave_sum(int v) {
  v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, true);   // row_shr:1
  v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, true);   // row_shr:2
  v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xe, true);   // row_shr:4
  v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xc, true);   // row_shr:8: lane 15 of a row holds the row's sum
  v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xa, 0xf, false);  // row_bcast:15 into rows 1 and 3
  v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xc, 0xf, false);  // row_bcast:31 into rows 2 and 3
  return __builtin_amdgcn_readlane(v, 63);
}
__device__ inline int wave_max(int v) {
  constexpr int lowest = -2147483647 - 1;
  v = max(v, __builtin_amdgcn_update_dpp(lowest, v, 0x111, 0xf, 0xf, false));
  v = max(v, __builtin_amdgcn_update_dpp(lowest, v, 0x112, 0xf, 0xf, false));
  v = max(v, __builtin_amdgcn_update_dpp(lowest, v, 0x114, 0xf, 0xe, false));
  v = max(v, __builtin_amdgcn_update_dpp(lowest, v, 0x118, 0xf, 0xc, false));
  v = max(v, __builtin_amdgcn_update_dpp(lowest, v, 0x142, 0xa, 0xf, false));
  v = max(v, __builtin_amdgcn_update_dpp(lowest, v, 0x143, 0xc, 0xf, false));
  return __builtin_amdgcn_readlane(v, 63);
}

// The cost behind an ordered_key (common.hpp): zero comes back as +0.0, every NaN as the canonical one.
__device__ inline float cost_of_key(uint32_t key) {
  if (key == 0xFFFFFFFFu) return __uint_as_float(0x7FC00000u);
  return __uint_as_float((key & 0x80000000u) ? key ^ 0x80000000u : ~key);
}

template <bool MASKED, int R, int U>
__device__ inline void scan_rows(const uint64_t* const (&row)[R], const int (&nw)[R], const uint64_t* mask_lds,
                                 RowScan (&out)[R]) {
  const int lane = threadIdx.x & 63;
  int total[R], last_w[R];
  uint64_t last_v[R];
  int nw_max = 0;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    total[r] = 0;
    last_w[r] = -1;
    last_v[r] = 0;
    nw_max = nw[r] > nw_max ? nw[r] : nw_max;
  }
  for (int w0 = lane * 2; w0 < nw_max; w0 += U * 128) {
    ulonglong2 v[R][U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int w = w0 + u * 128;
#pragma unroll
      for (int r = 0; r < R; ++r)
        v[r][u] = w < nw[r] ? *reinterpret_cast<const ulonglong2*>(row[r] + w) : make_ulonglong2(0ull, 0ull);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int w = w0 + u * 128;
      if (w < nw_max) {
        const uint64_t mx = MASKED ? mask_lds[w] : ~0ull;
        const uint64_t my = MASKED ? mask_lds[w + 1] : ~0ull;
#pragma unroll
        for (int r = 0; r < R; ++r) {
          const uint64_t ax = v[r][u].x & mx, ay = v[r][u].y & my;
          total[r] += __popcll(ax) + __popcll(ay);
          if (ax) { last_w[r] = w; last_v[r] = v[r][u].x; }
          if (ay) { last_w[r] = w + 1; last_v[r] = v[r][u].y; }
        }
      }
    }
  }
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int hi = wave_max(last_w[r]);
    out[r].total = wave_sum(total[r]);
    out[r].last_word = hi;
    // word w is held by lane (w / 2) % 64; that lane's own highest non-empty word is then w
    const int holder = hi < 0 ? 0 : (hi >> 1) & 63;
    const uint32_t lo = __builtin_amdgcn_readlane((int)(uint32_t)last_v[r], holder);
    const uint32_t up = __builtin_amdgcn_readlane((int)(uint32_t)(last_v[r] >> 32), holder);
    out[r].last_bits = hi < 0 ? 0ull : (((uint64_t)up << 32) | lo);
  }
}

template <bool MASKED>
__device__ inline RowScan scan_row(const uint64_t* __restrict__ row, int nw, const uint64_t* mask_lds) {
  const uint64_t* const rows[1] = {row};
  const int nws[1] = {nw};
  RowScan out[1];
  if (nw <= 512)
    scan_rows<MASKED, 1, 4>(rows, nws, mask_lds, out);
  else
    scan_rows<MASKED, 1, 8>(rows, nws, mask_lds, out);
  return out[0];
}

// ------------------------------------------------------------------ counts

// The highest non-empty word of a row (-1: the row is empty) by a walk from its top, 128 words a step, that ends at
// the first step that finds a bit: the witness passes want nothing else of a row, and in slot order a row's highest
// dominator lies a few dozen words below its own slot.  `total` is 1 or 0 (dominated or not), not the popcount.
__device__ inline RowScan scan_row_top(const uint64_t* __restrict__ row, int nw) {
  const int lane = threadIdx.x & 63;
  RowScan out;
  out.total = 0;
  out.last_word = -1;
  out.last_bits = 0ull;
  const int limit = (nw + 1) & ~1;
  for (int base = limit > 0 ? ((limit - 1) >> 7) << 7 : -1; base >= 0; base -= 128) {  // wave-uniform, from the top
    const int w = base + 2 * lane;
    const ulonglong2 v = w < limit ? *reinterpret_cast<const ulonglong2*>(row + w) : make_ulonglong2(0ull, 0ull);
    const uint64_t seen = __builtin_amdgcn_ballot_w64((v.x | v.y) != 0ull);
    if (seen != 0ull) {
      const int top = 63 - __builtin_clzll(seen);
      const int cand_word = v.y != 0ull ? w + 1 : w;
      const uint64_t cand_bits = v.y != 0ull ? v.y : v.x;
      out.total = 1;
      out.last_word = __builtin_amdgcn_readlane(cand_word, top);
      const uint32_t lo = __builtin_amdgcn_readlane((int)(uint32_t)cand_bits, top);
      const uint32_t hi = __builtin_amdgcn_readlane((int)(uint32_t)(cand_bits >> 32), top);
      out.last_bits = ((uint64_t)hi << 32) | lo;
      return out;
    }
  }
  return out;
}

// One wave per row (slot): popcount of the row = the domination count.  Rows with no dominator
// are rank 0 and form front 0, published both in slot space (for the passes) and in original-index
// space (for the listing).  witness[j] = the highest non-empty word of row j (-1 for ranked rows).
// Also fills the crowding-distance output with -inf when one is given.  Ranks are stored by
// original index.  need_counts = 0 (the peel that follows uses the witness pass): the rows are walked from the top
// only as far as their first dominator, and count[j] is 1 or 0.
__global__ __launch_bounds__(256) void count_kernel(const uint64_t* __restrict__ dom, int64_t wstride, int n,
                                                    const int* __restrict__ orig_of, int* __restrict__ count,
                                                    int* __restrict__ rank, int* __restrict__ witness,
                                                    uint64_t* __restrict__ front0_slot, uint64_t* __restrict__ front0_orig,
                                                    int* __restrict__ fsize, float* __restrict__ dist_fill,
                                                    const Ctrl* __restrict__ ctrl, const SortParam* __restrict__ param,
                                                    int need_counts) {
  if (ctrl->err != 0) return;  // the slot tables are not valid: leave front 0 empty, nothing gets peeled
  if (param->totals_valid != 0) return;  // count_from_totals_kernel does the work from what the dominance stage left
  __shared__ int block_found;
  if (threadIdx.x == 0) block_found = 0;
  __syncthreads();
  const int lane = threadIdx.x & 63;
  const int wave_in_block = threadIdx.x >> 6;
  const int waves = gridDim.x * (blockDim.x >> 6);
  int found = 0;
  for (int j = blockIdx.x * (blockDim.x >> 6) + wave_in_block; j < n; j += waves) {
    const RowScan r = need_counts ? scan_row<false>(dom + (int64_t)j * wstride, row_words(j), nullptr)
                                  : scan_row_top(dom + (int64_t)j * wstride, row_words(j));
    if (lane == 0) {
      const int o = orig_of[j];
      count[j] = r.total;
      rank[o] = r.total == 0 ? 0 : kRankUnset;
      witness[j] = r.last_word;
      if (dist_fill) dist_fill[o] = -INFINITY;
      if (r.total == 0) {
        atomicOr(reinterpret_cast<unsigned long long*>(front0_slot + (int64_t)(j >> 6) * kFrontStride), 1ull << (j & 63));
        atomicOr(reinterpret_cast<unsigned long long*>(front0_orig + (int64_t)(o >> 6) * kFrontStride), 1ull << (o & 63));
        ++found;
      }
    }
  }
  // one addition per block: a front 0 of thousands of rows would otherwise queue thousands of atomics on one word
  if (lane == 0 && found) atomicAdd(&block_found, found);
  __syncthreads();
  if (threadIdx.x == 0 && block_found) atomicAdd(fsize, block_found);
}

// The same outputs from total0[j] = popcount of row j and witness0[j] = its highest non-empty word (-1: none), which
// the order-based dominance kernel (prefix.hpp) accumulates while it builds the matrix: one thread per row, no row
// is read again.  Does nothing unless that kernel has run for this population.  A thread is slot j for what is
// kept by slot and original index j for what is kept by original index (through slot_of, the inverse of orig_of):
// both bitmaps of front 0 are then written a whole word per wave, with no atomics.
__global__ __launch_bounds__(256) void count_from_totals_kernel(const int* __restrict__ total0, const int* __restrict__ witness0,
                                                                int n, const int* __restrict__ slot_of, int* __restrict__ count,
                                                                int* __restrict__ rank, int* __restrict__ witness,
                                                                uint64_t* __restrict__ front0_slot,
                                                                uint64_t* __restrict__ front0_orig, int* __restrict__ fsize,
                                                                float* __restrict__ dist_fill, const Ctrl* __restrict__ ctrl,
                                                                const SortParam* __restrict__ param) {
  if (ctrl->err != 0 || param->totals_valid == 0) return;
  __shared__ int block_found;
  if (threadIdx.x == 0) block_found = 0;
  __syncthreads();
  // (few blocks, each walking through many rows: the blocks queue on the one word that holds the size of front 0)
  int found = 0;
  for (int j0 = blockIdx.x * blockDim.x + (threadIdx.x & ~63); j0 < n; j0 += gridDim.x * blockDim.x) {  // wave-uniform
    const int j = j0 + (threadIdx.x & 63);
    bool first = false, first_orig = false;
    if (j < n) {
      const int total = total0[j];
      count[j] = total;
      witness[j] = witness0[j];
      first = total == 0;
      first_orig = total0[slot_of[j]] == 0;  // the row whose original index is j
      rank[j] = first_orig ? 0 : kRankUnset;
      if (dist_fill) dist_fill[j] = -INFINITY;
    }
    const uint64_t members_orig = __builtin_amdgcn_ballot_w64(first_orig);
    // the 64 rows of a wave share one word of a bitmap: one store instead of up to 64 atomics
    const uint64_t members = __builtin_amdgcn_ballot_w64(first);
    if ((threadIdx.x & 63) == 0) {
      if (members_orig != 0ull) front0_orig[(int64_t)(j0 >> 6) * kFrontStride] = members_orig;
      if (members != 0ull) front0_slot[(int64_t)(j0 >> 6) * kFrontStride] = members;
      found += __popcll(members);
    }
  }
  if ((threadIdx.x & 63) == 0 && found) atomicAdd(&block_found, found);
  __syncthreads();
  if (threadIdx.x == 0 && block_found) atomicAdd(fsize, block_found);
}

// ------------------------------------------------------------ grid barrier

// Grid synchronisation with three roles, all through flag words and bounded polling:
//   block 0 ("master")   waits for the tally of every sweeping block, adds them up and publishes
//                        (generation << 32 | total) in `release`: one round trip both synchronises the
//                        sweepers and tells them the size of the front they just built;
//   block 1 ("lister")   follows `release` at its own pace (see peel_kernel) and is never waited for
//                        inside a pass;
//   blocks 2.. ("sweepers") publish (generation << 32 | rows found) in their own `arrive` slot and wait
//                        for `release`.
// No read-modify-write contention.  __syncthreads() makes every wave wait for its own outstanding
// memory operations (it carries a workgroup-scope fence) before the block's flag is written, and the
// data exchanged across the barrier is accessed coherently (see above), so no cache-wide fence is
// needed.  Every wait is bounded by `spin_limit` polls, after which the error flag is set and every
// role leaves its loop, so all waves always finish.
constexpr int kFirstSweeper = 2;
constexpr int kSharedListingRows = 8192;   // a final front 0 of more rows is listed by many blocks
constexpr int kSharedListingBlocks = 64;
constexpr int kFrontBuffers = 8;  // front bitmaps in rotation: the lister may lag the sweepers by 6 fronts

// Sweeper side.  Returns false after a timeout (here or elsewhere); *total_out = size of the new front.
__device__ inline bool sweeper_barrier(Ctrl* ctrl, unsigned gen, int block_tally, int* total_out, unsigned spin_limit,
                                       int* scratch) {
  __syncthreads();
  const unsigned long long want = (unsigned long long)gen << 32;
  if (threadIdx.x == 0) {
    coherent_store(&ctrl->arrive[blockIdx.x], want | (unsigned)block_tally);
    const unsigned long long* mine = &ctrl->release_copy[(blockIdx.x % kReleaseCopies) * 16];
    unsigned long long v = 0;
    const bool seen = bounded_wait([&] { return (v = coherent_load(mine)) >= want; }, spin_limit);
    if (!seen) coherent_store(&ctrl->err, kErrBarrierTimeout);
    scratch[0] = (int)(unsigned)(v & 0xFFFFFFFFull);
    scratch[1] = seen && v != kReleaseGiveUp;
  }
  __syncthreads();
  *total_out = scratch[0];
  const bool fine = scratch[1] != 0;
  __syncthreads();  // scratch is reused by the caller
  return fine;
}

// Master side: gathers the tallies of generation `gen` while one thread waits until the lister has
// cleared the bitmap that the coming pass will fill (`listed_needed` fronts cleared), then releases the
// sweepers.  After a timeout it releases them with the give-up word, so that nobody waits on.
__device__ inline bool master_barrier(Ctrl* ctrl, unsigned gen, int listed_needed, int* total_out, unsigned spin_limit,
                                      int* scratch) {
  const unsigned long long want = (unsigned long long)gen << 32;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int waves = blockDim.x >> 6;
  bool ok = true;
  int sum = 0;
  if (threadIdx.x == blockDim.x - 1)
    ok &= bounded_wait([&] { return coherent_load(&ctrl->listed) >= listed_needed; }, spin_limit);
  for (unsigned b = kFirstSweeper + threadIdx.x; b < gridDim.x; b += blockDim.x) {
    unsigned long long v = 0;
    ok &= bounded_wait([&] { return (v = coherent_load(&ctrl->arrive[b])) >= want; }, spin_limit);
    sum += (int)(unsigned)(v & 0xFFFFFFFFull);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off);
  const bool wave_ok = __builtin_amdgcn_ballot_w64(!ok) == 0ull;
  if (lane == 0) {
    scratch[wave] = sum;
    scratch[16 + wave] = wave_ok;
  }
  __syncthreads();
  int total = 0;
  bool fine = true;
  for (int v = 0; v < waves; ++v) {
    total += scratch[v];
    fine &= scratch[16 + v] != 0;
  }
  const unsigned long long word = fine ? (want | (unsigned)total) : kReleaseGiveUp;
  if (threadIdx.x < kReleaseCopies) coherent_store(&ctrl->release_copy[threadIdx.x * 16], word);
  if (threadIdx.x == kReleaseCopies) {
    if (!fine) coherent_store(&ctrl->err, kErrBarrierTimeout);
    coherent_store(&ctrl->release, word);
  }
  __syncthreads();  // scratch is reused by the next call
  *total_out = total;
  return fine;
}

// What the passes share: the matrix, the slot -> original index table, the output ranks (by
// original index) and the two bitmaps of the front being built.
struct PassCtx {
  const uint64_t* dom;
  int64_t wstride;
  int n;
  const int* orig_of;
  int* rank;
  uint64_t* next_slot;
  uint64_t* next_orig;
  int next_level;
};

__device__ inline void publish_ranked(const PassCtx& c, int slot, int orig) {
  c.rank[orig] = c.next_level;
  atomicOr(reinterpret_cast<unsigned long long*>(c.next_slot + (int64_t)(slot >> 6) * kFrontStride), 1ull << (slot & 63));
  atomicOr(reinterpret_cast<unsigned long long*>(c.next_orig + (int64_t)(orig >> 6) * kFrontStride), 1ull << (orig & 63));
}

// -------------------------------------------------------------- sweep pass

// count[j] -= popcount(row j & front) for every row of this wave's share that is still unranked.
// `front_lds` is the current front (slot space) copied to LDS.  Returns the number of rows this
// wave moved into the next front (in every lane).
__device__ inline int sweep_rows(const PassCtx& c, const uint64_t* front_lds, int* __restrict__ count, int first_row,
                                 int row_step) {
  const int lane = threadIdx.x & 63;
  int found = 0;
  int j = first_row;
  for (;;) {
    // the next two unranked rows of this wave's share: their loads are issued together
    int jr[2], cr[2];
    int have = 0;
    for (; j < c.n && have < 2; j += row_step) {
      const int cj = count[j];  // wave-uniform
      if (cj > 0) {
        jr[have] = j;
        cr[have] = cj;
        ++have;
      }
    }
    if (have == 0) break;
    if (have == 1) {
      jr[1] = jr[0];
      cr[1] = 0;
    }
    const uint64_t* const rows[2] = {c.dom + (int64_t)jr[0] * c.wstride, c.dom + (int64_t)jr[1] * c.wstride};
    const int nws[2] = {row_words(jr[0]), have == 2 ? row_words(jr[1]) : 0};
    RowScan r[2];
    if (nws[0] <= 512 && nws[1] <= 512)
      scan_rows<true, 2, 4>(rows, nws, front_lds, r);
    else
      scan_rows<true, 2, 8>(rows, nws, front_lds, r);
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      if (q < have && r[q].total) {
        const int left = cr[q] - r[q].total;
        if (lane == 0) {
          count[jr[q]] = left;
          if (left == 0) publish_ranked(c, jr[q], c.orig_of[jr[q]]);
        }
        found += left == 0;
      }
    }
  }
  return found;
}

// ------------------------------------------------------------ witness pass

// Every unranked row remembers the highest word of its row that held an unranked dominator when it
// was last looked at (the "witness": word index + word value, kept in the registers of the lane that
// owns the row, so the common case touches no memory at all).  A pass only tests that word against
// the bitmap of unranked rows; when none of its dominators is left the wave rescans the row against
// the bitmap and either finds the new highest word or ranks the row.  In slot order the highest
// dominator is almost always the one ranked last, so nearly every rescan is the one that ranks the
// row.  Same results as the count formulation.
constexpr int kWitnessChunks = 4;  // a wave owns up to 4 x 64 rows

struct WitnessState {
  int word[kWitnessChunks];        // witness word index, -1 = ranked (or no row)
  int orig[kWitnessChunks];        // original index of the row
  uint64_t bits[kWitnessChunks];   // that word of the row
};

// Rows are dealt to the sweeping waves round-robin (row = wave + index * waves): rows of
// neighbouring slots enter the same fronts, and this keeps each front's rescans spread over all waves.
__device__ inline void witness_load(WitnessState& st, const PassCtx& c, const int* __restrict__ witness, int first_row,
                                    int row_step) {
  const int lane = threadIdx.x & 63;
#pragma unroll
  for (int ch = 0; ch < kWitnessChunks; ++ch) {
    const int64_t j64 = (int64_t)first_row + (int64_t)(ch * 64 + lane) * row_step;
    const bool have = j64 < c.n;
    const int j = have ? (int)j64 : 0;
    st.word[ch] = have ? witness[j] : -1;
    st.orig[ch] = have ? c.orig_of[j] : 0;
    st.bits[ch] = st.word[ch] >= 0 ? c.dom[(int64_t)j * c.wstride + st.word[ch]] : 0ull;
  }
}

// The witness passes only need the highest word of a row that still holds an unranked dominator, and
// that word: found with one lane-mask per 128 words (which lanes saw an unranked dominator), the highest
// lane of the highest non-empty mask, and three lane reads -- no cross-lane reduction through the LDS
// permute unit, whose six dependent steps per row made the rescan the longest part of a pass.
// Lane l holds words 2 l + 128 u and 2 l + 128 u + 1, so later lanes and later u mean higher words.
template <int R, int U>
__device__ inline void scan_rows_highest(const uint64_t* const (&row)[R], const int (&nw)[R], const uint64_t* mask_lds,
                                         RowScan (&out)[R]) {
  const int lane = threadIdx.x & 63;
  int nw_max = 0;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    out[r].total = 0;  // not computed here
    out[r].last_word = -1;
    out[r].last_bits = 0ull;
    nw_max = nw[r] > nw_max ? nw[r] : nw_max;
  }
  for (int w0 = lane * 2; w0 - lane * 2 < nw_max; w0 += U * 128) {  // wave-uniform trip count
    ulonglong2 v[R][U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int w = w0 + u * 128;
#pragma unroll
      for (int r = 0; r < R; ++r)
        v[r][u] = w < nw[r] ? *reinterpret_cast<const ulonglong2*>(row[r] + w) : make_ulonglong2(0ull, 0ull);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int w = w0 + u * 128;
      const bool inside = w < nw_max;
      const uint64_t mx = inside ? mask_lds[w] : 0ull;
      const uint64_t my = inside ? mask_lds[w + 1] : 0ull;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const uint64_t ax = v[r][u].x & mx, ay = v[r][u].y & my;
        const uint64_t seen = __builtin_amdgcn_ballot_w64((ax | ay) != 0ull);
        if (seen != 0ull) {  // wave-uniform; a later (r, u) of the same row overrides an earlier one
          const int top = 63 - __builtin_clzll(seen);
          const int cand_word = ay != 0ull ? w + 1 : w;
          const uint64_t cand_bits = ay != 0ull ? v[r][u].y : v[r][u].x;
          out[r].last_word = __builtin_amdgcn_readlane(cand_word, top);
          const uint32_t lo = __builtin_amdgcn_readlane((int)(uint32_t)cand_bits, top);
          const uint32_t hi = __builtin_amdgcn_readlane((int)(uint32_t)(cand_bits >> 32), top);
          out[r].last_bits = ((uint64_t)hi << 32) | lo;
        }
      }
    }
  }
}

// Rescan of up to four rows against the bitmap of unranked rows, all loads in flight together.
// Entries from `cnt` on repeat entry 0 and are ignored.
__device__ inline void scan_up_to_four(const uint64_t* const (&rows)[4], const int (&nws)[4], int cnt, const uint64_t* alive_lds,
                                       RowScan (&r)[4]) {
  const bool short_rows = nws[0] <= 512 && nws[1] <= 512 && nws[2] <= 512 && nws[3] <= 512;
  if (cnt > 2 && short_rows) {
    scan_rows_highest<4, 4>(rows, nws, alive_lds, r);
  } else {
    // (unrolled, so that the arrays are indexed by constants: indexed at run time they would live in scratch memory,
    // a round trip to memory in every rescan)
#pragma unroll
    for (int q0 = 0; q0 < 4; q0 += 2) {
      if (q0 >= cnt) break;
      const uint64_t* const two[2] = {rows[q0], rows[q0 + 1]};
      const int nw2[2] = {nws[q0], nws[q0 + 1]};
      RowScan r2[2];
      if (short_rows)
        scan_rows_highest<2, 4>(two, nw2, alive_lds, r2);
      else
        scan_rows_highest<2, 8>(two, nw2, alive_lds, r2);
      r[q0] = r2[0];
      r[q0 + 1] = r2[1];
    }
  }
}

// `on_ranked(slot, original index)` is called, by the lane that owns the row, for every row that enters the
// front being built.
template <class OnRanked>
__device__ inline int witness_rows(WitnessState& st, const PassCtx& c, const uint64_t* alive_lds, int first_row,
                                   int row_step, OnRanked on_ranked) {
  const int lane = threadIdx.x & 63;
  int found = 0;
  int stat_rows = 0, stat_rounds = 0;
#pragma unroll
  for (int ch = 0; ch < kWitnessChunks; ++ch) {
    const bool need = st.word[ch] >= 0 && (st.bits[ch] & alive_lds[st.word[ch] < 0 ? 0 : st.word[ch]]) == 0;
    uint64_t todo = __builtin_amdgcn_ballot_w64(need);
    while (todo) {
      // up to four rows per round: their loads overlap
      int l[4], jrow[4], nws[4];
      const uint64_t* rows[4];
      int cnt = 0;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const bool have = todo != 0;
        if (have) {
          l[q] = __ffsll((unsigned long long)todo) - 1;
          todo &= todo - 1;
          ++cnt;
        } else {
          l[q] = l[0];
        }
        jrow[q] = first_row + (ch * 64 + l[q]) * row_step;
        rows[q] = c.dom + (int64_t)jrow[q] * c.wstride;
        nws[q] = row_words(jrow[q]);
      }
      stat_rows += cnt;
      ++stat_rounds;
      RowScan r[4];
      scan_up_to_four(rows, nws, cnt, alive_lds, r);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        if (q < cnt) {
          if (lane == l[q]) {
            st.word[ch] = r[q].last_word;
            st.bits[ch] = r[q].last_bits;
            if (r[q].last_word < 0) on_ranked(jrow[q], st.orig[ch]);
          }
          found += r[q].last_word < 0;
        }
      }
    }
  }
  EVX_RESCAN(c.next_level - 1, stat_rows, stat_rounds);
  (void)stat_rows;
  (void)stat_rounds;
  return found;
}

// The same pass with the rescans of a whole block pooled: the rows that lost their witness are queued
// in LDS and dealt to the block's waves four at a time, so that a wave that owns five such rows does not
// take two rounds while its neighbours idle (with 20 rows per wave that happens somewhere in almost
// every pass, and everybody waits for the slowest wave).  q_row / q_word / q_bits hold one entry per
// queued row (q_word: in, the number of leading words to scan; out, the new witness word); *q_n must be
// zero on entry.
template <class OnRanked>
__device__ inline void witness_rows_pooled(WitnessState& st, const PassCtx& c, const uint64_t* alive_lds, int first_row,
                                           int row_step, int* q_n, int* q_row, int* q_word, uint64_t* q_bits, int q_capacity,
                                           OnRanked on_ranked) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int waves = blockDim.x >> 6;
  int mine[kWitnessChunks];
#pragma unroll
  for (int ch = 0; ch < kWitnessChunks; ++ch) {
    const bool need = st.word[ch] >= 0 && (st.bits[ch] & alive_lds[st.word[ch] < 0 ? 0 : st.word[ch]]) == 0;
    mine[ch] = -1;
    if (need) {
      const int idx = atomicAdd(q_n, 1);
      if (idx < q_capacity) {
        q_row[idx] = first_row + (ch * 64 + lane) * row_step;
        q_word[idx] = st.word[ch];  // words from the dead witness upwards hold no unranked dominator
        mine[ch] = idx;
      }
    }
  }
  lds_barrier();
  EVX_TRACE_POOL(c.next_level - 1, 2);
  const int total = min(*q_n, q_capacity);
  for (int base = wave * 4; base < total; base += waves * 4) {
    const int cnt = min(4, total - base);
    int jrow[4], nws[4];
    const uint64_t* rows[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      jrow[q] = q_row[base + (q < cnt ? q : 0)];
      rows[q] = c.dom + (int64_t)jrow[q] * c.wstride;
      nws[q] = q_word[base + (q < cnt ? q : 0)];  // scan below the dead witness word only
    }
    RowScan r[4];
    const uint64_t* const four[4] = {rows[0], rows[1], rows[2], rows[3]};
    scan_up_to_four(four, nws, cnt, alive_lds, r);
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      if (q < cnt && lane == q) {
        q_word[base + q] = r[q].last_word;
        q_bits[base + q] = r[q].last_bits;
      }
    }
  }
  EVX_TRACE_POOL(c.next_level - 1, 3);
  lds_barrier();
#pragma unroll
  for (int ch = 0; ch < kWitnessChunks; ++ch) {
    if (mine[ch] >= 0) {
      st.word[ch] = q_word[mine[ch]];
      st.bits[ch] = q_bits[mine[ch]];
      if (st.word[ch] < 0) on_ranked(first_row + (ch * 64 + lane) * row_step, st.orig[ch]);
    }
  }
}

// Block-wide listing of the set bits of `front` (nwords words, LDS) in ascending order into
// perm[base ...]; the words are words first_word ... of the whole bitmap.  `scratch` holds at least
// blockDim.x / 64 ints.
template <bool LDS_BARRIERS = false>  // true: the barriers inside order LDS traffic only (see lds_barrier)
__device__ inline void list_front(const uint64_t* front_lds, int nwords, int* __restrict__ perm, int base, int* scratch,
                                  int first_word = 0) {
  // each thread owns a contiguous slice of words so that the order is ascending
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int per = (nwords + blockDim.x - 1) / blockDim.x;
  const int w_begin = threadIdx.x * per;
  const int w_end = min(nwords, w_begin + per);
  int mine = 0;
  for (int w = w_begin; w < w_end; ++w) mine += __popcll(front_lds[w]);
  // inclusive scan inside the wave, then across the (few) waves through LDS
  int incl = mine;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const int up = __shfl_up(incl, off);
    if (lane >= off) incl += up;
  }
  if (lane == 63) scratch[wave] = incl;
  if (LDS_BARRIERS) lds_barrier(); else __syncthreads();
  int pos = base + incl - mine;
  for (int v = 0; v < wave; ++v) pos += scratch[v];
  for (int w = w_begin; w < w_end; ++w) {
    uint64_t bits = front_lds[w];
    while (bits) {
      const int b = __ffsll((unsigned long long)bits) - 1;
      perm[pos++] = (first_word + w) * 64 + b;
      bits &= bits - 1;
    }
  }
  if (LDS_BARRIERS) lds_barrier(); else __syncthreads();
}

// --------------------------------------------------------- persistent peel

// fronts_slot / fronts_orig: kFrontBuffers bitmaps of nwords words each (kFrontStride apart); front r lives in buffer
// r % kFrontBuffers of both (slot space for the passes, original-index space for the listing).
// fsize[0] and buffer 0 come from count_kernel; the other buffers must be zero.
// perm may be null when only ranks are wanted.
// Stops as soon as the fronts built so far hold stop_count rows (stop_count = n ranks everything).
// use_witness selects the witness pass (needs 2 * nwords words of LDS and at most
// kWitnessChunks * 64 rows per sweeping wave) instead of the popcount sweep (nwords words of LDS).
// The host launches at least three blocks (master, lister, one sweeper), all resident at once.
__global__ __launch_bounds__(kPeelThreads) void peel_kernel(const uint64_t* __restrict__ dom, int64_t wstride, int nwords,
                                                             int n, const int* __restrict__ orig_of, int* __restrict__ count,
                                                             int* __restrict__ rank, uint64_t* __restrict__ fronts_slot,
                                                             uint64_t* __restrict__ fronts_orig, int* __restrict__ fsize,
                                                             int* __restrict__ perm, int* __restrict__ fstart,
                                                             Ctrl* __restrict__ ctrl, int stop_count, unsigned spin_limit,
                                                             const int* __restrict__ witness, int use_witness) {
  extern __shared__ uint64_t front_lds[];  // nwords words (nwords is even: rows are padded to 128),
                                           // followed by nwords more (unranked rows) in witness mode
  __shared__ int scratch[kPeelThreads];
  if (coherent_load(&ctrl->err) != 0) return;  // an earlier kernel of this call gave up

  if (blockIdx.x == 0) {
    // ---- master: nothing but the barrier
    int level = 0, ranked = 0;
    int size = coherent_load(&fsize[0]);
    for (;;) {
      if (size <= 0 || ranked + size >= stop_count) break;
      ranked += size;
      ++level;
      // pass `level` fills the bitmaps that held front level + 1 - kFrontBuffers: that front and all
      // before it must have been listed and cleared
      if (!master_barrier(ctrl, (unsigned)level, level + 2 - kFrontBuffers, &size, spin_limit, scratch)) break;
    }
    return;
  }

  if (blockIdx.x == 1) {
    // ---- lister: for each finished front, in order: list its rows (ascending original index) into
    // perm, which makes perm a stable ordering by rank; record where the front starts; clear the
    // bitmaps of the front before it for reuse.
    int ranked = 0;
    for (int level = 0;; ++level) {
      if (level > 0) {
        const unsigned long long want = (unsigned long long)level << 32;
        if (threadIdx.x == 0) {
          unsigned long long v = 0;
          if (!bounded_wait([&] { return (v = coherent_load(&ctrl->release)) >= want || coherent_load(&ctrl->err) != 0; },
                            spin_limit))
            coherent_store(&ctrl->err, kErrBarrierTimeout);
          scratch[48] = coherent_load(&ctrl->err) | (v == kReleaseGiveUp);
        }
        __syncthreads();
        const bool bad = scratch[48] != 0;
        __syncthreads();
        if (bad) return;
        // The sweepers have now finished the pass that read front level-1: its bitmaps can be cleared.
        uint64_t* prev_slot = fronts_slot + (int64_t)((level - 1) % kFrontBuffers) * nwords * kFrontStride;
        uint64_t* prev_orig = fronts_orig + (int64_t)((level - 1) % kFrontBuffers) * nwords * kFrontStride;
        for (int w = threadIdx.x; w < nwords; w += blockDim.x) {
          coherent_store(&prev_slot[(int64_t)w * kFrontStride], (uint64_t)0);
          coherent_store(&prev_orig[(int64_t)w * kFrontStride], (uint64_t)0);
        }
      }
      const uint64_t* cur = fronts_orig + (int64_t)(level % kFrontBuffers) * nwords * kFrontStride;
      int mine = 0;
      for (int w = threadIdx.x; w < nwords; w += blockDim.x) {
        const uint64_t fw = coherent_load(&cur[(int64_t)w * kFrontStride]);
        front_lds[w] = fw;
        mine += __popcll(fw);
      }
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) mine += __shfl_xor(mine, off);
      if ((threadIdx.x & 63) == 0) scratch[32 + (threadIdx.x >> 6)] = mine;
      __syncthreads();  // also waits for the clearing stores of this block's waves
      int size = 0;
      for (int v = 0; v < (int)(blockDim.x >> 6); ++v) size += scratch[32 + v];
      if (threadIdx.x == 0) coherent_store(&ctrl->listed, level);  // fronts 0 .. level-1 are cleared
      const bool last = size <= 0 || ranked + size >= stop_count;
      // a front 0 that ends the peel is listed by the sweepers together (they have nothing else to do, and it
      // may hold most of a large population)
      const bool shared_listing = level == 0 && last && size > kSharedListingRows && gridDim.x > kFirstSweeper;
      if (perm && !shared_listing) list_front(front_lds, nwords, perm, ranked, scratch);
      if (threadIdx.x == 0) {
        fstart[level] = ranked;
        if (level > 0) fsize[level] = size;
        if (last) {
          fstart[level + 1] = ranked + size;
          ctrl->nfronts = level + 1;
          ctrl->worst = level;
          ctrl->worst_start = ranked;
          ctrl->nv = size;
          ctrl->need = stop_count - ranked;
          ctrl->passes = level;
        }
      }
      if (last) return;
      ranked += size;
      __syncthreads();
    }
  }

  // ---- sweepers
  uint64_t* alive_lds = front_lds + nwords;
  const int waves_per_block = blockDim.x >> 6;
  const int sweep_blocks = gridDim.x - kFirstSweeper;
  const int sweep_block = (int)blockIdx.x - kFirstSweeper;
  const int row_step = sweep_blocks * waves_per_block;
  const int first_row = sweep_block * waves_per_block + (threadIdx.x >> 6);
  PassCtx c;
  c.dom = dom;
  c.wstride = wstride;
  c.n = n;
  c.orig_of = orig_of;
  c.rank = rank;
  WitnessState st;
  int size = coherent_load(&fsize[0]);  // size of front `level`
  if (size <= 0 || size >= stop_count) {  // front 0 already holds every row asked for: no pass
    if (perm && size > kSharedListingRows) {
      // list it: the first sweeping blocks take a slice of the bitmap (original-index space) each, after adding
      // up the rows of the words before their slice
      const int listers = min(sweep_blocks, kSharedListingBlocks);
      if (sweep_block < listers) {
        const int per = (nwords + listers - 1) / listers;
        const int w_begin = min(nwords, sweep_block * per), w_end = min(nwords, w_begin + per);
        int before = 0;
        for (int w = threadIdx.x; w < w_end; w += blockDim.x) {
          const uint64_t fw = coherent_load(&fronts_orig[(int64_t)w * kFrontStride]);
          if (w < w_begin)
            before += __popcll(fw);
          else
            front_lds[w - w_begin] = fw;
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) before += __shfl_xor(before, off);
        if ((threadIdx.x & 63) == 0) scratch[32 + (threadIdx.x >> 6)] = before;
        __syncthreads();
        before = 0;
        for (int v = 0; v < (int)(blockDim.x >> 6); ++v) before += scratch[32 + v];
        __syncthreads();
        list_front(front_lds, w_end - w_begin, perm, before, scratch, w_begin);
      }
    }
    return;
  }
  if (use_witness) {
    witness_load(st, c, witness, first_row, row_step);
    for (int w = threadIdx.x; w < nwords; w += blockDim.x) {
      const int lo = w * 64;
      alive_lds[w] = lo + 64 <= n ? ~0ull : (lo >= n ? 0ull : ((1ull << (n - lo)) - 1ull));
    }
  }
  int level = 0;
  int ranked = 0;  // rows in fronts 0 .. level-1
  for (;;) {
    EVX_TRACE(level, 0);
    if (size <= 0 || ranked + size >= stop_count) break;  // size 0 cannot happen for 1 <= stop_count <= n
    const uint64_t* cur = fronts_slot + (int64_t)(level % kFrontBuffers) * nwords * kFrontStride;
    c.next_slot = fronts_slot + (int64_t)((level + 1) % kFrontBuffers) * nwords * kFrontStride;
    c.next_orig = fronts_orig + (int64_t)((level + 1) % kFrontBuffers) * nwords * kFrontStride;
    c.next_level = level + 1;
    // the words of the front just finished, four per thread in flight at once
    for (int w0 = threadIdx.x; w0 < nwords; w0 += 4 * blockDim.x) {
      uint64_t fw[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int w = w0 + u * blockDim.x;
        fw[u] = w < nwords ? coherent_load(&cur[(int64_t)w * kFrontStride]) : 0ull;
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int w = w0 + u * blockDim.x;
        if (w < nwords) {
          if (use_witness)
            alive_lds[w] &= ~fw[u];
          else
            front_lds[w] = fw[u];
        }
      }
    }
    __syncthreads();
    EVX_TRACE(level, 1);
    const int found = use_witness ? witness_rows(st, c, alive_lds, first_row, row_step,
                                                 [&](int slot, int orig) { publish_ranked(c, slot, orig); })
                                  : sweep_rows(c, front_lds, count, first_row, row_step);
    EVX_TRACE(level, 2);
    // every lane of a wave holds that wave's tally
    if ((threadIdx.x & 63) == 0) scratch[threadIdx.x >> 6] = found;
    __syncthreads();
    int tally = 0;
    for (int v = 0; v < waves_per_block; ++v) tally += scratch[v];
    EVX_TRACE(level, 3);
    ranked += size;
    ++level;
    if (!sweeper_barrier(ctrl, (unsigned)level, tally, &size, spin_limit, scratch + 64)) break;
  }
}

// ------------------------------------------- persistent peel, record protocol

// A pass of peel_kernel is a chain of dependent device-coherent exchanges (front bitmap load, rescan,
// publish, arrive -> master, release -> sweepers).  This kernel removes three of them for populations
// of moderate size: every sweeping block announces the rows it has just ranked in a RECORD of its own,
// and every block reads the records of all blocks.  A record is a row of 8-byte units, each written and
// read with one relaxed atomic access and each carrying the low 16 bits of the pass number in its top
// bits, so a unit says by itself whether it belongs to the pass awaited: unit 0 holds the number of rows
// and two slots, the others three slots each (16-bit slots, kRecNil for none), and a writer always
// writes all its units.  Seeing every unit of a generation is therefore both the grid barrier and the
// exchange of the new front, in one hop, with no master.  The units of one generation are few (8 KB):
// a block that polls more than that per round waits on its own uncached loads.  A block that ranks more
// rows than fit its record publishes them through the front bitmaps (as peel_kernel does), waits for
// those atomics and flags the overflow in unit 0; in such a pass the readers also load the bitmap.
// Records live in a ring of kRecRing generations; the lister (block 0) follows at its own pace, builds
// each front in original-index space from the records, lists it into perm and recycles bitmaps;
// `listed` keeps the sweepers from lapping it.  All waits are bounded.
constexpr int kRecThreads = 512;
constexpr int kRecUnits = 1024;  // units of one generation = sweepers x units per record
constexpr int kRecRing = 8;      // == kFrontBuffers: a generation's record slot and bitmap buffer recycle together
constexpr int kRecLoads = kRecUnits / kRecThreads;
// Populations of 65 535 rows and more (the wide layout: two slots per unit) have fronts of thousands of rows, and a
// workgroup whose rows of a front do not fit its record sends everybody to the bitmaps in memory for that pass
// (200 000 x 3: 2000 rows a front, 128 sweepers with room for 15 each).  Their generations hold four times the
// units: room for 63 rows per workgroup.
constexpr int kRecUnitsWide = 4 * kRecUnits;
constexpr uint32_t kRecOverflowNarrow = 0x8000u;  // in the count field: the rows are in the bitmaps, not in the record
static_assert(kRecRing == kFrontBuffers, "records and bitmaps are recycled by the same counter");

// Two layouts of a unit.  Narrow (populations of fewer than 65535 rows): generation : 16 | three 16-bit fields;
// wide (fewer than 2^24 - 1 rows): generation : 16 | two 24-bit fields.  Unit 0 of a record carries the count
// (with the overflow flag in its top bit) in its first field, every other field is a slot or "none" (all ones).
template <bool WIDE>
struct RecFormat {
  static constexpr int kFields = WIDE ? 2 : 3;
  static constexpr int kBits = WIDE ? 24 : 16;
  static constexpr uint32_t kMask = (1u << kBits) - 1u;
  static constexpr uint32_t kNil = kMask;
  static constexpr uint32_t kOverflow = 1u << (kBits - 1);
  // Slots that a record of `units` units can carry.
  __device__ static int capacity(int units) { return kFields - 1 + kFields * (units - 1); }
  __device__ static unsigned long long pack(unsigned gen, const uint32_t (&f)[3]) {
    unsigned long long v = (unsigned long long)(gen & 0xFFFFu) << 48;
#pragma unroll
    for (int k = 0; k < kFields; ++k) v |= (unsigned long long)(f[k] & kMask) << (kBits * (kFields - 1 - k));
    return v;
  }
  // The unit that thread i (< units) of the writer stores: list = (slot, original index) pairs, cnt of them.
  __device__ static unsigned long long unit_for(unsigned gen, int i, const int* list, int cnt, bool overflow) {
    auto slot_at = [&](int k) { return (!overflow && k < cnt) ? (uint32_t)list[2 * k] : kNil; };
    uint32_t f[3] = {kNil, kNil, kNil};
    if (i == 0) {
      f[0] = overflow ? (kOverflow | (uint32_t)cnt) : (uint32_t)cnt;
#pragma unroll
      for (int k = 1; k < kFields; ++k) f[k] = slot_at(k - 1);
    } else {
#pragma unroll
      for (int k = 0; k < kFields; ++k) f[k] = slot_at(kFields * i - 1 + k);
    }
    return pack(gen, f);
  }
  // Calls on_count(count, overflow) for a unit 0 and on_slot(slot) for every slot a unit carries.
  template <class OnCount, class OnSlot>
  __device__ static void read(unsigned long long v, bool is_first, OnCount on_count, OnSlot on_slot) {
#pragma unroll
    for (int k = 0; k < kFields; ++k) {
      const uint32_t field = (uint32_t)(v >> (kBits * (kFields - 1 - k))) & kMask;
      if (k == 0 && is_first)
        on_count((int)(field & ~kOverflow), (field & kOverflow) != 0u);
      else if (field != kNil)
        on_slot((int)field);
    }
  }
};

// Waits until the kRecLoads units of generation `gen` that this thread reads are all present (and, for
// the thread that is given a counter, until *listed >= listed_needed).  False after a timeout or when
// another block has given up.  Only what is still missing is loaded again: a block's uncached loads are
// served one after the other, so every extra polling load delays the one that matters (two rounds in
// flight at once, or records four times this size, each cost more than a microsecond per pass).
template <int kRecLoads>
__device__ inline bool poll_record_units(const unsigned long long* gen_units, int used_units, unsigned gen,
                                         unsigned long long (&v)[kRecLoads], const int* listed, int listed_needed,
                                         const int* err, unsigned spin_limit) {
  const unsigned long long* mine = gen_units + threadIdx.x;
  unsigned pending = 0u;
#pragma unroll
  for (int k = 0; k < kRecLoads; ++k) {
    // units past the last record are never written: they read as "no slot"
    if ((int)threadIdx.x + k * kRecThreads < used_units)
      pending |= 1u << k;
    else
      v[k] = ~0ull;
  }
  bool waiting_listed = listed != nullptr;
  WaitBound bound(spin_limit);
  for (unsigned spins = 0;; ++spins) {
    int seen_listed = 0;
#pragma unroll
    for (int k = 0; k < kRecLoads; ++k)
      if (pending & (1u << k)) v[k] = coherent_load(&mine[k * kRecThreads]);
    if (waiting_listed) seen_listed = coherent_load(listed);
#pragma unroll
    for (int k = 0; k < kRecLoads; ++k)
      if ((pending & (1u << k)) && (unsigned)(v[k] >> 48) == (gen & 0xFFFFu)) pending &= ~(1u << k);
    if (waiting_listed && seen_listed >= listed_needed) waiting_listed = false;
    if (pending == 0u && !waiting_listed) return true;
    if (bound.expired(spins)) return false;
    if ((spins & 63u) == 63u && coherent_load(err) != 0) return false;
  }
}

template <bool WIDE>
__global__ __launch_bounds__(kRecThreads) void peel_records_kernel(
    const uint64_t* __restrict__ dom, int64_t wstride, int nwords, int n, const int* __restrict__ orig_of,
    int* __restrict__ rank, uint64_t* __restrict__ fronts_slot, uint64_t* __restrict__ fronts_orig, int* __restrict__ fsize,
    int* __restrict__ perm, int* __restrict__ fstart, Ctrl* __restrict__ ctrl, int stop_count, unsigned spin_limit,
    const int* __restrict__ witness, unsigned long long* __restrict__ records, int sweepers, int list_capacity) {
  extern __shared__ uint64_t rec_lds[];  // nwords words: unranked rows (sweepers) / the front being listed (lister);
                                         // then, per row a block can own (list_capacity): the rescan queue
                                         // (result bits, row, result word) and the (slot, original index) pairs
                                         // of the rows just ranked
  __shared__ int sh[32];
  if (coherent_load(&ctrl->err) != 0) return;
  constexpr int kRecUnits = WIDE ? evx::kRecUnitsWide : evx::kRecUnits;  // (units of a generation, in this kernel)
  constexpr int kRecLoads = kRecUnits / kRecThreads;
  int units = 1;  // per record: the largest power of two that gives every sweeper a record
  while (units * 2 * sweepers <= kRecUnits) units *= 2;
  const int tid = threadIdx.x;

  if (blockIdx.x == 0) {
    // ---- lister
    uint64_t* front_lds = rec_lds;
    int ranked = 0;
    // The bitmaps of a front in memory are written by the count stage (front 0) and by sweepers whose rows of a front
    // did not fit their record; nobody else touches them, so those of a front whose records all fitted are still
    // clear.  (Clearing them whatever they held made the lister the slowest block from 65 535 rows on: two stores
    // per 128-byte line of two buffers, 17 of its 21 us per front at 200 000 rows, and the sweepers wait for it.)
    bool prev_written = true;
    for (int level = 0;; ++level) {
      int size = 0;
      if (level == 0) {
        const uint64_t* cur = fronts_orig;  // buffer 0, filled by count_kernel
        int mine = 0;
        for (int w = tid; w < nwords; w += blockDim.x) {
          const uint64_t fw = coherent_load(&cur[(int64_t)w * kFrontStride]);
          front_lds[w] = fw;
          mine += __popcll(fw);
        }
        if (tid == 0) sh[1] = 0;
        __syncthreads();
        if (mine) atomicAdd(&sh[1], mine);
        __syncthreads();
        size = sh[1];
      } else {
        EVX_TRACE(level, 0);
        for (int w = tid; w < nwords; w += blockDim.x) front_lds[w] = 0ull;
        if (tid == 0) {
          sh[1] = 0;
          sh[2] = 0;
        }
        __syncthreads();
        unsigned long long v[kRecLoads];
        const unsigned gen = (unsigned)level;
        if (!poll_record_units(records + (size_t)(gen % kRecRing) * kRecUnits, sweepers * units, gen, v, nullptr, 0, &ctrl->err,
                               spin_limit)) {
          coherent_store(&ctrl->err, kErrBarrierTimeout);
          atomicOr(&sh[2], 2);
        } else {
          // (the original indices of all slots of this thread's units are fetched together: one after the other, with
          // the addition to the bitmap in between, they were a memory round trip each)
          constexpr int kFields = RecFormat<WIDE>::kFields;
          int slots[kRecLoads * kFields];
#pragma unroll
          for (int k = 0; k < kRecLoads; ++k) {
#pragma unroll
            for (int q = 0; q < kFields; ++q) slots[k * kFields + q] = -1;
            if (tid + k * kRecThreads >= sweepers * units) continue;  // past the last record
            const int i = (tid + k * kRecThreads) & (units - 1);
            int at = 0;
            RecFormat<WIDE>::read(
                v[k], i == 0,
                [&](int count, bool overflow) {
                  atomicAdd(&sh[1], count);
                  if (overflow) atomicOr(&sh[2], 1);
                },
                [&](int slot) { slots[k * kFields + at++] = slot; });
          }
          int origs[kRecLoads * kFields];
#pragma unroll
          for (int e = 0; e < kRecLoads * kFields; ++e) origs[e] = slots[e] >= 0 ? orig_of[slots[e]] : -1;
#pragma unroll
          for (int e = 0; e < kRecLoads * kFields; ++e)
            if (origs[e] >= 0) atomicOr(reinterpret_cast<unsigned long long*>(&front_lds[origs[e] >> 6]), 1ull << (origs[e] & 63));
        }
        __syncthreads();
        EVX_TRACE(level, 1);
        if (sh[2] & 2) return;
        size = sh[1];
        if (sh[2] & 1) {
          const uint64_t* cur = fronts_orig + (int64_t)(level % kFrontBuffers) * nwords * kFrontStride;
          for (int w = tid; w < nwords; w += blockDim.x) front_lds[w] |= coherent_load(&cur[(int64_t)w * kFrontStride]);
        }
        // every sweeper has published generation `level`, so it has finished with the bitmaps of front level-1
        if (prev_written) {
          uint64_t* prev_slot = fronts_slot + (int64_t)((level - 1) % kFrontBuffers) * nwords * kFrontStride;
          uint64_t* prev_orig = fronts_orig + (int64_t)((level - 1) % kFrontBuffers) * nwords * kFrontStride;
          for (int w = tid; w < nwords; w += blockDim.x) {
            coherent_store(&prev_slot[(int64_t)w * kFrontStride], (uint64_t)0);
            coherent_store(&prev_orig[(int64_t)w * kFrontStride], (uint64_t)0);
          }
        }
        prev_written = (sh[2] & 1) != 0;
      }
      __syncthreads();  // also waits for the clearing stores of this block's waves
      EVX_TRACE(level, 2);
      if (tid == 0) coherent_store(&ctrl->listed, level);  // records <= level consumed, bitmaps < level cleared
      const bool last = size <= 0 || ranked + size >= stop_count;
      // a front 0 that ends the peel is listed by the sweepers together (see peel_kernel)
      const bool shared_listing = level == 0 && last && size > kSharedListingRows;
      if (perm && !shared_listing) list_front(front_lds, nwords, perm, ranked, sh + 8);
      EVX_TRACE(level, 3);
      if (tid == 0) {
        fstart[level] = ranked;
        if (level > 0) fsize[level] = size;
        if (last) {
          fstart[level + 1] = ranked + size;
          ctrl->nfronts = level + 1;
          ctrl->worst = level;
          ctrl->worst_start = ranked;
          ctrl->nv = size;
          ctrl->need = stop_count - ranked;
          ctrl->passes = level;
        }
      }
      if (last) return;
      ranked += size;
      __syncthreads();
    }
  }

  // ---- sweepers
  uint64_t* alive_lds = rec_lds;
  uint64_t* q_bits = rec_lds + nwords;
  int* found = reinterpret_cast<int*>(q_bits + list_capacity);
  int* q_row = found + 2 * list_capacity;
  int* q_word = q_row + list_capacity;
  const int waves_per_block = blockDim.x >> 6;
  const int sb = (int)blockIdx.x - 1;
  const int row_step = sweepers * waves_per_block;
  const int first_row = sb * waves_per_block + (tid >> 6);
  PassCtx c;
  c.dom = dom;
  c.wstride = wstride;
  c.n = n;
  c.orig_of = orig_of;
  c.rank = rank;
  int size = coherent_load(&fsize[0]);  // size of front `level`
  if (size <= 0 || size >= stop_count) {  // front 0 already holds every row asked for: no pass
    if (perm && size > kSharedListingRows) {
      // list it: the first sweeping blocks take a slice of the bitmap (original-index space) each, after adding
      // up the rows of the words before their slice
      const int listers = min(sweepers, kSharedListingBlocks);
      if (sb < listers) {
        const int per = (nwords + listers - 1) / listers;
        const int w_begin = min(nwords, sb * per), w_end = min(nwords, w_begin + per);
        int before = 0;
        for (int w = tid; w < w_end; w += blockDim.x) {
          const uint64_t fw = coherent_load(&fronts_orig[(int64_t)w * kFrontStride]);
          if (w < w_begin)
            before += __popcll(fw);
          else
            rec_lds[w - w_begin] = fw;
        }
        if (tid == 0) sh[0] = 0;
        __syncthreads();
        if (before) atomicAdd(&sh[0], before);
        __syncthreads();
        list_front(rec_lds, w_end - w_begin, perm, sh[0], sh + 8, w_begin);
      }
    }
    return;
  }
  WitnessState st;
  witness_load(st, c, witness, first_row, row_step);
  for (int w = tid; w < nwords; w += blockDim.x) {
    const int lo = w * 64;
    const uint64_t all = lo + 64 <= n ? ~0ull : (lo >= n ? 0ull : ((1ull << (n - lo)) - 1ull));
    alive_lds[w] = all & ~coherent_load(&fronts_slot[(int64_t)w * kFrontStride]);  // minus front 0 (buffer 0)
  }
  // The counters of a pass live in sh[4 p .. 4 p + 3], p = the parity of the pass: [0] rows this block ranks,
  // [1] rows all blocks rank, [2] bit 0: some block overflowed its record, bit 1: give up, [3] rows queued
  // for a rescan.  Those of the next pass are cleared in the middle of this one (between two barriers that
  // the pass needs anyway), so that a pass neither starts nor ends with a barrier of its own.
  if (tid < 8) sh[tid] = 0;
  __syncthreads();
  int level = 0;
  int ranked = 0;  // rows in fronts 0 .. level-1
  for (;;) {
    if (size <= 0 || ranked + size >= stop_count) break;
    ranked += size;
    ++level;  // this pass builds front `level`
    const unsigned gen = (unsigned)level;
    c.next_slot = fronts_slot + (int64_t)(level % kFrontBuffers) * nwords * kFrontStride;
    c.next_orig = fronts_orig + (int64_t)(level % kFrontBuffers) * nwords * kFrontStride;
    c.next_level = level;
    int* const cnts = sh + 4 * (level & 1);
    int* const next_cnts = sh + 4 * ((level + 1) & 1);
    EVX_TRACE(level - 1, 0);
    witness_rows_pooled(st, c, alive_lds, first_row, row_step, &cnts[3], q_row, q_word, q_bits, list_capacity, [&](int slot, int orig) {
      rank[orig] = level;
      const int k = atomicAdd(&cnts[0], 1);
      if (k < list_capacity) {
        found[2 * k] = slot;
        found[2 * k + 1] = orig;
      }
    });
    lds_barrier();  // the list of ranked rows is complete (the rank stores need not be)
    EVX_TRACE(level - 1, 1);
    const int cnt = cnts[0];
    if (tid < 4) next_cnts[tid] = 0;  // last read before the barrier above, first used after the one below
    unsigned long long* mine = records + (size_t)(gen % kRecRing) * kRecUnits + (size_t)sb * units;
    if (cnt <= RecFormat<WIDE>::capacity(units)) {
      if (tid < units) coherent_store(&mine[tid], RecFormat<WIDE>::unit_for(gen, tid, found, cnt, false));
    } else {
      for (int e = tid; e < cnt; e += blockDim.x) {
        const int slot = found[2 * e], orig = found[2 * e + 1];
        atomicOr(reinterpret_cast<unsigned long long*>(c.next_slot + (int64_t)(slot >> 6) * kFrontStride), 1ull << (slot & 63));
        atomicOr(reinterpret_cast<unsigned long long*>(c.next_orig + (int64_t)(orig >> 6) * kFrontStride), 1ull << (orig & 63));
      }
      __syncthreads();  // every wave has waited for its own atomics
      if (tid < units) coherent_store(&mine[tid], RecFormat<WIDE>::unit_for(gen, tid, found, cnt, true));
    }
    // the records of everybody: barrier and front exchange in one.  Thread 0 also makes sure that the
    // lister has recycled what generation level + 1 will overwrite.
    EVX_TRACE(level - 1, 2);
    unsigned long long v[kRecLoads];
    const bool fine = poll_record_units(records + (size_t)(gen % kRecRing) * kRecUnits, sweepers * units, gen, v,
                                        tid == 0 ? &ctrl->listed : nullptr, level + 2 - kRecRing, &ctrl->err, spin_limit);
    EVX_TRACE(level - 1, 3);
    if (!fine) {
      coherent_store(&ctrl->err, kErrBarrierTimeout);
      atomicOr(&cnts[2], 2);
    } else {
#pragma unroll
      for (int k = 0; k < kRecLoads; ++k) {
        if (tid + k * kRecThreads >= sweepers * units) continue;  // past the last record
        const int i = (tid + k * kRecThreads) & (units - 1);
        RecFormat<WIDE>::read(
            v[k], i == 0,
            [&](int count, bool overflow) {
              atomicAdd(&cnts[1], count);
              if (overflow) atomicOr(&cnts[2], 1);
            },
            [&](int slot) { atomicAnd(reinterpret_cast<unsigned long long*>(&alive_lds[slot >> 6]), ~(1ull << (slot & 63))); });
      }
    }
    lds_barrier();  // the bitmap of unranked rows and the counters of the pass are complete
    const int flags = cnts[2];
    size = cnts[1];
    if (flags & 2) break;
    if (flags & 1) {  // the same in every thread
      const uint64_t* cur = c.next_slot;
      for (int w = tid; w < nwords; w += blockDim.x) alive_lds[w] &= ~coherent_load(&cur[(int64_t)w * kFrontStride]);
      lds_barrier();
    }
  }
}

}  // namespace evx
