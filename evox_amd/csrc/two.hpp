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
// 880 of them at 200 000 rows).
//
// The scan of a round runs through the workgroups like a bucket brigade: workgroup b owns a run of slots, receives
// the minimum over the remaining rows before its run from workgroup b - 1 and hands min(that, its own minimum) on to
// workgroup b + 1.  The rounds of different workgroups overlap: F fronts over B workgroups take F rounds of the last
// workgroup plus what the B hand-overs put between the first workgroup's start and the last one's, not F * B.  A
// workgroup only ever waits for the one before it (and, when it is a whole ring of rounds ahead, for the one after
// it); all waits are bounded.  Rows holding a NaN neither dominate nor are dominated: rank 0, and they take no part.
//
// A round inside a workgroup is ONE barrier: every wave leaves the prefix minimum of its rows in LDS, and behind the
// barrier every wave reads the sixteen wave minima and the incoming minimum and ranks its own rows.  Everything that
// talks to other workgroups happens beside that, in single lanes of two waves, because a wave waits for its memory
// operations in the order of their issue (a load that has to see another workgroup's store takes half a
// microsecond, most of a round, and a write-through store longer):
//   * the first wave holds no rows.  Right behind the barrier of round q - 1 its first lane loads the word of round q
//     -- tag checked, loaded again while it is not there -- and leaves it in LDS for the barrier of round q; the load
//     takes as long as the other waves rank their rows.  This wave stores nothing;
//   * the first lane of the last wave publishes: behind the barrier of round r it counts what round r - 1 ranked,
//     stores the word of round r for the next workgroup and the progress counter for the one before, and decides
//     whether the workgroup is done (seen by all waves behind the next barrier).  It loads nothing but, once every
//     ring of rounds, the progress of the workgroup after.  The ranks stay in registers until the kernel ends, so the
//     other waves store nothing inside the loop either.
// A workgroup runs about 1.3 us behind the one before it (the time a stored word takes to be seen and loaded).  A
// round takes 0.65 us -- instruction issue: fifteen waves of some eighty instructions on four SIMDs; half as many
// waves with twice the rows each take as long, since one or two waves per SIMD wait nine clocks for every dependent
// instruction instead of four -- where the two barriers and the one thread between them of an earlier form of this
// kernel took 1.25: that thread waited for its own write-through stores and for loads issued a round earlier.
// Measured and no faster: words asked for one to six rounds ahead (into accumulation registers, so that the compiler
// places no wait at the end of the loop body), by the wave without rows or by lanes of waves that also hold rows (a
// word that is not there yet costs such a wave a second load on top of its rows: 0.85 us per round); falling back on
// purpose (a sleep after the first late word).
#pragma once

#include "peel.hpp"

namespace evx {

constexpr int kTwoThreads = 1024;
constexpr int kTwoWaves = kTwoThreads / 64;
constexpr int kTwoPerThread = 4;                             // consecutive slots per thread
constexpr int kTwoChunk = (kTwoThreads - 64) * kTwoPerThread;  // slots per workgroup: the first wave holds none
constexpr int kTwoMaxBlocks = 512;  // (two workgroups of 1024 threads per compute unit)
constexpr int64_t kTwoMaxRows = (int64_t)kTwoChunk * kTwoMaxBlocks;
constexpr int kTwoRing = 256;                                // rounds of a workgroup's outgoing stream that are kept
constexpr int kTwoRingStride = kTwoRing + 16;                // words per workgroup: the ring, then its progress counter on a line of its own
constexpr int kTwoPublisher = kTwoThreads - 64;              // the thread that stores
constexpr int kTwoRounds = 4;                                // Ctrl.reserved[kTwoRounds]: the rounds of the last workgroup (every rank up to the cut is below it)
constexpr uint32_t kTwoNone = 0xFFFFFFFFu;                   // "no remaining row": larger than every image of a number
// A word of a ring: the minimum in the low half; in the high half bit 31 "nothing remains in this workgroup or before
// it", bits 30:29 the generation of the ring slot (1..3, 0 = never written: the ring starts zeroed), bits 28:0 the
// number of rows that this workgroup and those before it have ranked in the rounds before the word's round.
constexpr unsigned kTwoEnd = 0x80000000u;
constexpr unsigned kTwoTagShift = 29;
constexpr unsigned kTwoCountMask = (1u << kTwoTagShift) - 1u;
__device__ inline unsigned two_tag(int round) { return (unsigned)((round / kTwoRing) % 3) + 1u; }
__device__ inline unsigned two_tag_of(unsigned long long word) { return ((unsigned)(word >> 32) >> kTwoTagShift) & 3u; }
static_assert(kTwoMaxRows <= (int64_t)kTwoCountMask, "the count of ranked rows must fit its field");
static_assert(kTwoWaves <= 16, "the wave minima are reduced inside rows of sixteen lanes");
// flags of an incoming word as the waves see it in LDS
constexpr uint32_t kTwoInEnded = 1u;  // nothing remains before this workgroup, from this round on
constexpr uint32_t kTwoInStop = 2u;   // leave now: a wait ran out, or enough rows are ranked everywhere

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
// (by original index), rank 0 for rows holding a NaN, and the -inf fill of the distances.  stop_count >= n: every front
// is peeled.  stop_count < n: the peeling may end once the fronts so far hold stop_count rows -- the last workgroup,
// which sees the count of all workgroups a round late, raises a flag that the others find a few rounds later;
// rows not ranked by then are left at kRankUnset, and a front after the one that holds the stop_count-th row may be
// ranked in part.  Only first rows of a key count (copies and rows with a NaN do not): the peeling never ends before
// the stop_count-th row has its rank, and goes through all fronts where copies make up the difference.
// ring: gridDim.x * kTwoRingStride words, zero at the start of the call.  blockIdx.z: one of several populations in the
// launch, whose buffers lie ws_step bytes apart (each population a chain of gridDim.x workgroups of its own).
__global__ __launch_bounds__(kTwoThreads) void two_peel_kernel(const float* __restrict__ xs1_sorted, const float* __restrict__ xs2_sorted,
                                                               const uint32_t* __restrict__ kid, const int* __restrict__ orig_of,
                                                               int n, int* __restrict__ rank, float* __restrict__ dist_fill,
                                                               Ctrl* __restrict__ ctrl, unsigned long long* __restrict__ ring,
                                                               unsigned spin_limit, int stop_count, int64_t ws_step) {
  to_population(ws_step, xs1_sorted, xs2_sorted, kid, orig_of, rank, dist_fill, ctrl, ring);
  __shared__ __attribute__((aligned(16))) uint32_t wave_min_lds[2][16];  // by the parity of the round; entries from kTwoWaves on stay "none"
  // by the parity of the round: incoming minimum, rows ranked before this workgroup, flags (these three from the lane
  // that loads), "the workgroup leaves behind this round's barrier" (from the lane that publishes)
  __shared__ __attribute__((aligned(16))) uint32_t in_lds[2][4];
  __shared__ int ranked_lds[2];    // rows this workgroup ranked in a round, by the parity of the round
  __shared__ int unranked_lds[kTwoWaves];
  if (coherent_load(&ctrl->err) != 0) return;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int b = blockIdx.x;
  const bool last_block = b == (int)gridDim.x - 1;
  unsigned long long* my_ring = ring + (size_t)b * kTwoRingStride;
  const unsigned long long* up_ring = ring + (size_t)(b > 0 ? b - 1 : 0) * kTwoRingStride;
  int* my_progress = reinterpret_cast<int*>(my_ring + kTwoRing);  // rounds of the stream before that this workgroup has taken in
  const int* down_progress = reinterpret_cast<const int*>(ring + (size_t)(last_block ? b : b + 1) * kTwoRingStride + kTwoRing);
  // "enough rows are ranked": in the spare words behind the last workgroup's ring (whose progress counter nobody reads)
  int* const enough_flag = reinterpret_cast<int*>(ring + (size_t)(gridDim.x - 1) * kTwoRingStride + kTwoRing + 8);
  const bool may_stop = stop_count < n;
  // ---- this thread's slots
  uint32_t v[kTwoPerThread];
  int orig[kTwoPerThread];   // -1: the slot takes no part
  int rk[kTwoPerThread];
  int unranked = 0;
  {
    const int s0 = b * kTwoChunk + (tid - 64) * kTwoPerThread;
#pragma unroll
    for (int e = 0; e < kTwoPerThread; ++e) {
      const int s = s0 + e;
      v[e] = kTwoNone;
      orig[e] = -1;
      rk[e] = kRankUnset;
      if (wave > 0 && s < n) {
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
  if (tid == 0) {
    ranked_lds[0] = 0;
    ranked_lds[1] = 0;
    in_lds[0][3] = 0u;
    in_lds[1][3] = 0u;
  }
  if (tid < 32) wave_min_lds[tid >> 4][tid & 15] = kTwoNone;  // (the first wave's entries stay that way)
  unranked = wave_sum(unranked);
  if (lane == 0) unranked_lds[wave] = unranked;
  __syncthreads();
  const bool publisher = tid == kTwoPublisher;
  const bool receiver = tid == 0;
  // (publisher) rows of this workgroup without a rank, rows ranked so far by this workgroup, the progress of the
  // workgroup after this one as last read
  int left = 0, done_here = 0, down_seen = 0;
  if (publisher)
    for (int w = 0; w < kTwoWaves; ++w) left += unranked_lds[w];
  const bool lower = (lane & 15) < wave;  // this lane's entry of the wave minima belongs to a wave before this one
  // Takes in the word of round q (before: the flags and the count that round q - 1 saw) and leaves it in LDS for the
  // barrier of round q.
  auto receive = [&](int q, uint32_t flags_before, uint32_t count_before) {
    uint32_t in = kTwoNone, count = count_before, flags = flags_before & kTwoInEnded;
    if (!(flags & kTwoInEnded) || may_stop) {
      const unsigned long long* slot = up_ring + (q % kTwoRing);
      // (the word and the flag in flight together)
      unsigned long long word = (flags & kTwoInEnded) ? 0ull : coherent_load(slot);
      bool enough = may_stop && coherent_load(enough_flag) != 0;
      bool failed = false;
      if (!enough && !(flags & kTwoInEnded)) {
        const unsigned tag = two_tag(q);
        if (two_tag_of(word) != tag) {  // not there yet: the workgroup before is less than a store and a load ahead
          WaitBound bound(spin_limit);
          for (unsigned spins = 0;; ++spins) {
            word = coherent_load(slot);
            if (two_tag_of(word) == tag) break;
            if (may_stop && (spins & 3u) == 3u && coherent_load(enough_flag) != 0) {  // (the workgroup before may have left on it)
              enough = true;
              break;
            }
            if (bound.expired(spins) || ((spins & 63u) == 63u && coherent_load(&ctrl->err) != 0)) {
              failed = true;
              break;
            }
          }
        }
        if (!failed && !enough) {
          in = (uint32_t)word;
          count = (unsigned)(word >> 32) & kTwoCountMask;
          if ((unsigned)(word >> 32) & kTwoEnd) flags |= kTwoInEnded;
        }
      }
      if (failed) coherent_store(&ctrl->err, kErrBarrierTimeout);
      if (failed || enough) flags |= kTwoInStop;
    }
    in_lds[q & 1][0] = in;
    in_lds[q & 1][1] = count;
    in_lds[q & 1][2] = flags;
  };
  if (receiver) receive(0, b == 0 ? kTwoInEnded : 0u, 0u);
  int round = 0;
  for (;; ++round) {
    const int par = round & 1;
    // ---- the minimum of this thread's remaining rows, of the wave's rows up to this lane
    uint32_t incl = kTwoNone;
    if (wave > 0) {
      uint32_t tmin = kTwoNone;
#pragma unroll
      for (int e = 0; e < kTwoPerThread; ++e) tmin = min(tmin, v[e]);
      incl = wave_prefix_min(tmin);
      if (lane == 63) wave_min_lds[par][wave] = incl;
    }
    EVX_TRACE(round, 0);
    lds_barrier();
    EVX_TRACE(round, 1);
    const uint4 in_word = *reinterpret_cast<const uint4*>(in_lds[par]);
    const uint32_t in = in_word.x, count_in = in_word.y, flags = in_word.z;
    if (((flags & kTwoInStop) | in_word.w) != 0u) break;  // (the same for every wave: written before the barrier)
    if (wave == 0) {  // the wave without rows: the word of the next round
      if (receiver) receive(round + 1, flags, count_in);
      EVX_TRACE(round, 3);
      continue;
    }
    const uint32_t wave_min = wave_min_lds[par][lane & 15];
    // ---- what stands before this wave: the minimum over the wave minima of the waves before, reduced inside every
    // row of sixteen lanes (all lanes get it)
    uint32_t before = lower ? wave_min : kTwoNone;
    before = min(before, (uint32_t)__builtin_amdgcn_update_dpp((int)kTwoNone, (int)before, 0x128, 0xf, 0xf, false));  // row_ror:8
    before = min(before, (uint32_t)__builtin_amdgcn_update_dpp((int)kTwoNone, (int)before, 0x124, 0xf, 0xf, false));  // row_ror:4
    before = min(before, (uint32_t)__builtin_amdgcn_update_dpp((int)kTwoNone, (int)before, 0x122, 0xf, 0xf, false));  // row_ror:2
    before = min(before, (uint32_t)__builtin_amdgcn_update_dpp((int)kTwoNone, (int)before, 0x121, 0xf, 0xf, false));  // row_ror:1
    before = min(before, in);
    before = min(before, (uint32_t)__builtin_amdgcn_update_dpp((int)kTwoNone, (int)incl, 0x138, 0xf, 0xf, false));  // wave_shr:1
    // ---- the rows that are strict prefix minima form the front of this round
    int ranked = 0;  // (of the whole wave)
#pragma unroll
    for (int e = 0; e < kTwoPerThread; ++e) {
      const uint32_t mine_e = v[e];
      const bool front = mine_e < before;  // no remaining row before it is no worse in both objectives
      ranked += __popcll(__builtin_amdgcn_ballot_w64(front));
      rk[e] = front ? round : rk[e];
      v[e] = front ? kTwoNone : mine_e;
      before = min(before, mine_e);
    }
    if (ranked != 0 && lane == 0) atomicAdd(&ranked_lds[par], ranked);  // (read behind the next barrier)
    EVX_TRACE(round, 2);
    if (wave == kTwoPublisher / 64) {
      // the minimum of the workgroup
      uint32_t local = wave_min;
      local = min(local, (uint32_t)__builtin_amdgcn_update_dpp((int)kTwoNone, (int)local, 0x128, 0xf, 0xf, false));  // row_ror:8
      local = min(local, (uint32_t)__builtin_amdgcn_update_dpp((int)kTwoNone, (int)local, 0x124, 0xf, 0xf, false));  // row_ror:4
      local = min(local, (uint32_t)__builtin_amdgcn_update_dpp((int)kTwoNone, (int)local, 0x122, 0xf, 0xf, false));  // row_ror:2
      local = min(local, (uint32_t)__builtin_amdgcn_update_dpp((int)kTwoNone, (int)local, 0x121, 0xf, 0xf, false));  // row_ror:1
      if (publisher) {
        const int before_round = ranked_lds[par ^ 1];  // what round - 1 has ranked
        ranked_lds[par ^ 1] = 0;
        left -= before_round;
        done_here += before_round;
        const int done = (int)count_in + done_here;
        const bool ended_before = (flags & kTwoInEnded) != 0u;
        // the stream ends with the round in which neither this workgroup nor those before it have a row left
        const bool ends_here = ended_before && left == 0;
        bool stop_next = ends_here;
        if (last_block) {
          if (may_stop && done >= stop_count) {  // enough rows ranked everywhere, as of the round before this one
            coherent_store(enough_flag, 1);
            stop_next = true;
          }
        } else {
          bool go = true;
          if (round >= kTwoRing && down_seen < round - kTwoRing + 1) {  // (the slot still holds round - kTwoRing: has the next workgroup taken it in?)
            WaitBound bound(spin_limit);
            for (unsigned spins = 0;; ++spins) {
              down_seen = coherent_load(down_progress);
              if (down_seen >= round - kTwoRing + 1) break;
              if (may_stop && (spins & 3u) == 3u && coherent_load(enough_flag) != 0) {
                go = false;
                break;
              }
              if (bound.expired(spins) || ((spins & 63u) == 63u && coherent_load(&ctrl->err) != 0)) {
                coherent_store(&ctrl->err, kErrBarrierTimeout);
                go = false;
                break;
              }
            }
          }
          if (go)
            coherent_store(my_ring + (round % kTwoRing),
                           ((unsigned long long)((ends_here ? kTwoEnd : 0u) | (two_tag(round) << kTwoTagShift) | (unsigned)done) << 32) | min(in, local));
          else
            stop_next = true;
        }
        if (!ended_before) coherent_store(my_progress, round + 1);
        in_lds[par ^ 1][3] = stop_next ? 1u : 0u;
      }
    }
  }
  if (last_block && publisher) ctrl->reserved[kTwoRounds] = round;  // (for the sort of the ranks: how many bits they have)
  // ---- the ranks, kept in registers so far; rows that no round has reached (the peeling ended early, or a wait ran
  // out) stay unset
#pragma unroll
  for (int e = 0; e < kTwoPerThread; ++e)
    if (orig[e] >= 0) rank[orig[e]] = rk[e];
}

// After the brigade: the rows of a key take the rank of the key's first row.
__global__ __launch_bounds__(256) void two_finish_kernel(const uint32_t* __restrict__ kid, const int* __restrict__ orig_of,
                                                         const float* __restrict__ xs1_sorted, const float* __restrict__ xs2_sorted,
                                                         int n, int* __restrict__ rank, const Ctrl* __restrict__ ctrl, int64_t ws_step) {
  to_population(ws_step, kid, orig_of, xs1_sorted, xs2_sorted, rank, ctrl);
  if (ctrl->err != 0) return;
  for (int s = blockIdx.x * blockDim.x + threadIdx.x; s < n; s += gridDim.x * blockDim.x) {
    const int first = (int)kid[s];
    if (first == s) continue;
    const float a1 = xs1_sorted[s], a2 = xs2_sorted[s];
    if (a1 != a1 || a2 != a2) continue;  // rank 0, written by the brigade
    rank[orig_of[s]] = rank[orig_of[first]];
  }
}

// After the listing (perm = rows by (rank, original index) up to the cut front and beyond; behind the fronts that every
// workgroup has been through, rows of later fronts and rows without a rank follow in no particular order): where every
// front starts, and the front that holds the stop_count-th row, as the control block
// describes it for the kernels that order it.  Every front up to that one is complete; later ones may be ranked in
// part, their starts mean nothing.
__global__ __launch_bounds__(256) void two_bounds_kernel(const int* __restrict__ perm, const int* __restrict__ rank, int n,
                                                         int* __restrict__ fstart, Ctrl* __restrict__ ctrl, int stop_count, int64_t ws_step) {
  to_population(ws_step, perm, rank, fstart, ctrl);
  if (ctrl->err != 0) return;
  const int worst = rank[perm[stop_count - 1]];
  for (int p = blockIdx.x * blockDim.x + threadIdx.x; p < n; p += gridDim.x * blockDim.x) {
    const int r = rank[perm[p]];
    const int r_before = p > 0 ? rank[perm[p - 1]] : -1;
    if (r != r_before) {  // position p opens front r and closes front r_before
      if (r != kRankUnset) fstart[r] = p;
      if (r_before == worst) fstart[worst + 1] = p;  // (whatever follows the cut front: the next one, a later one ranked in part, rows without a rank)
      if (r == worst) {
        ctrl->worst = worst;
        ctrl->nfronts = worst + 1;
        ctrl->passes = worst;
        ctrl->worst_start = p;
        ctrl->need = stop_count - p;
      }
    }
    if (p == n - 1 && r != kRankUnset) fstart[r + 1] = n;
  }
}

// ... and the sizes of the fronts, from their starts (one small launch behind the one above).
__global__ __launch_bounds__(256) void two_sizes_kernel(const int* __restrict__ perm, const int* __restrict__ rank, int n,
                                                        const int* __restrict__ fstart, int* __restrict__ fsize,
                                                        Ctrl* __restrict__ ctrl, int* __restrict__ rank_until_out, int64_t ws_step) {
  to_population(ws_step, perm, rank, fstart, fsize, ctrl, rank_until_out);  // (the ranks up to the cut lie in the workspaces too)
  if (ctrl->err != 0) return;
  const int worst = ctrl->worst;
  const int last = rank[perm[n - 1]];
  const int fronts = last == kRankUnset ? worst + 1 : last + 1;
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
