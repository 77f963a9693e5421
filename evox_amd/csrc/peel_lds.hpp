// Front peeling with the dominated-by bit matrix resident in LDS.
//
// Reference semantics (the same as peel.hpp):
//   count = A.sum(dim=0); front = count == 0                    src/evox/operators/selection/non_dominate.py:188-192
//   while the front is not empty: rank[front] = level; the rows whose dominators are now all ranked form the next
//   front                                                       non_dominate.py:29-59, :161-169
//
// The lower triangle of a population of up to about 24 000 rows (20 000 rows: 25.6 MB) fits the LDS of the device
// (256 compute units x 160 KB) but not that of a few workgroups, and a pass of the peeling is a chain of dependent
// steps -- which rows have lost their last unranked dominator, tell everybody -- whose length is what a selection
// waits for.  With the rows in memory the first step costs a memory round trip per pass (and the slowest of them
// counts); here every sweeping workgroup copies its rows into LDS once, counting them on the way (which is the
// column sum of the reference and replaces a pass of its own over the matrix), and a pass touches memory only to
// exchange the new front: the record protocol of peel_records_kernel, one hop, no master.
//
// Rows are dealt to the waves of all sweeping workgroups round-robin (row = global wave + k * waves), a wave's
// k-th row belongs to its lane k; the lane keeps the row's witness (the highest word that held an unranked
// dominator, see peel.hpp) in registers.  Front 0 goes through the records like every other front (generation =
// level + 1, so that a cleared record never looks current).
#pragma once

#include "peel.hpp"

namespace evx {

constexpr int kLdsPeelThreads = 512;  // (1024 threads: the rows are copied 2 us sooner, the first exchange takes 2 us longer)
constexpr int kLdsPeelRowsPerWave = 64;  // one row per lane
constexpr int kLdsPeelMaxRowsPerBlock = kLdsPeelRowsPerWave * (kLdsPeelThreads / 64);

// Bytes of dynamic LDS for a grid of `sweepers` sweeping workgroups (an upper bound over the workgroups: as if
// every wave's k-th row were the longest k-th row of any wave), 0 when a wave would own more than 64 rows.
__host__ inline size_t lds_peel_bytes(int n, int nwords, int sweepers) {
  const int waves = kLdsPeelThreads / 64;
  const int64_t step = (int64_t)sweepers * waves;
  const int64_t per_wave = (n + step - 1) / step;
  if (per_wave > kLdsPeelRowsPerWave) return 0;
  const int64_t rows_cap = per_wave * waves;
  int64_t words = 0;
  for (int64_t k = 0; k < per_wave; ++k) {
    int64_t j = (k + 1) * step - 1;
    if (j > n - 1) j = n - 1;
    words += waves * (int64_t)((((j >> 6) + 2) & ~1ll));
  }
  // unranked-row bitmap, row offsets (padded to 16 bytes), (slot, original index) pairs of the rows just ranked, rows
  const int64_t sweeper = 8 * (int64_t)nwords + 4 * ((rows_cap + 4) & ~3ll) + 8 * rows_cap + 8 * words;
  // the lister: the bitmap of the front being listed, a listing offset per word and the slot -> original index
  // table (16 bits per row)
  const int64_t lister = 12 * (int64_t)nwords + 2 * (int64_t)n;
  return (size_t)(sweeper > lister ? sweeper : lister);
}

// Every generation of records is written kRecCopies times: a sweeping workgroup reads the copy of its die (workgroup
// b runs on die b % 8) and the lister a copy of its own -- 255 workgroups polling the same 8 KB queue on the few
// memory channels that hold it (a load of the lister from a polled copy took 1.9 us).
constexpr int kRecSweeperCopies = 8;
constexpr int kRecCopies = kRecSweeperCopies + 1;
constexpr size_t kLdsPeelRecordUnits = (size_t)kRecRing * kRecCopies * kRecUnits;

// Waits until the two neighbouring units of generation `gen` that this thread reads (units 2 t and 2 t + 1, one
// 16-byte load: every 8-byte unit says by itself whether it is current, so the load need not be atomic as a whole)
// are present, and thread `listed`'s counter has reached listed_needed.  False after a timeout or when another
// workgroup has given up.
__device__ inline bool poll_record_pair(const unsigned long long* gen_units, int used_units, unsigned gen,
                                        unsigned long long (&v)[2], const int* listed, int listed_needed, const int* err,
                                        unsigned spin_limit) {
  typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
  const int idx = 2 * (int)threadIdx.x;
  const bool have = idx < used_units;  // used_units is even
  v[0] = v[1] = ~0ull;                 // units past the last record are never written: they read as "no slot"
  bool waiting = have, waiting_listed = listed != nullptr;
  const unsigned long long* mine = gen_units + (have ? idx : 0);
  WaitBound bound(spin_limit);
  for (unsigned spins = 0;; ++spins) {
    if (waiting) {
      u32x4 r;
      asm volatile("global_load_dwordx4 %0, %1, off sc1\n\ts_waitcnt vmcnt(0)" : "=v"(r) : "v"(mine) : "memory");
      if ((r.y >> 16) == (gen & 0xFFFFu) && (r.w >> 16) == (gen & 0xFFFFu)) {
        v[0] = ((unsigned long long)r.y << 32) | r.x;
        v[1] = ((unsigned long long)r.w << 32) | r.z;
        waiting = false;
      }
    }
    if (waiting_listed && coherent_load(listed) >= listed_needed) waiting_listed = false;
    if (!waiting && !waiting_listed) return true;
    if (bound.expired(spins)) return false;
    if ((spins & 63u) == 63u && coherent_load(err) != 0) return false;
  }
}

// Highest word below `nw` of a row held in LDS that still has a bit in `alive`; -1 when there is none.  The row
// starts on a 16-byte boundary; the same result in every lane.
__device__ inline void lds_row_highest(const uint64_t* row, int nw, const uint64_t* alive, int& word_out, uint64_t& bits_out) {
  const int lane = threadIdx.x & 63;
  word_out = -1;
  bits_out = 0ull;
  const int limit = (nw + 1) & ~1;
  for (int base = limit > 0 ? ((limit - 1) >> 7) << 7 : -1; base >= 0; base -= 128) {  // wave-uniform, from the top
    const int w = base + 2 * lane;
    ulonglong2 v = make_ulonglong2(0ull, 0ull), a = make_ulonglong2(0ull, 0ull);
    if (w < limit) {
      v = *reinterpret_cast<const ulonglong2*>(row + w);
      a = *reinterpret_cast<const ulonglong2*>(alive + w);
    }
    const uint64_t ax = v.x & a.x, ay = v.y & a.y;
    const uint64_t seen = __builtin_amdgcn_ballot_w64((ax | ay) != 0ull);
    if (seen != 0ull) {
      const int top = 63 - __builtin_clzll(seen);
      const int cand_word = ay != 0ull ? w + 1 : w;
      const uint64_t cand_bits = ay != 0ull ? v.y : v.x;
      word_out = __builtin_amdgcn_readlane(cand_word, top);
      const uint32_t lo = __builtin_amdgcn_readlane((int)(uint32_t)cand_bits, top);
      const uint32_t hi = __builtin_amdgcn_readlane((int)(uint32_t)(cand_bits >> 32), top);
      bits_out = ((uint64_t)hi << 32) | lo;
      return;
    }
  }
}

// (sort key, original index below 32 768) as one number that a double holds exactly, and the key back out of it.
__device__ inline double tail_composite(uint32_t key, int orig) {
  return (double)(((unsigned long long)key << 15) | (unsigned)orig);
}
__device__ inline uint32_t tail_composite_key(double c) { return (uint32_t)((unsigned long long)c >> 15); }
// (as instructions: the compiler's own maximum first makes sure that neither operand is a signalling NaN)
__device__ inline double max_f64(double a, double b) {
  double r;
  asm("v_max_f64 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}
__device__ inline double min_f64(double a, double b) {
  double r;
  asm("v_min_f64 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}
// Lanes that share one item of the last front's scans when a workgroup of kLdsPeelThreads has `items` of them.
__device__ inline int tail_group_lanes(int items) {
  return items * 64 <= kLdsPeelThreads ? 64 : items * 32 <= kLdsPeelThreads ? 32 : 16;
}
__device__ inline double shfl_xor_f64(double v, int off) {
  const unsigned long long b = (unsigned long long)__double_as_longlong(v);
  const unsigned long long o = ((unsigned long long)__shfl_xor((unsigned)(b >> 32), off) << 32) | __shfl_xor((unsigned)b, off);
  return __longlong_as_double((long long)o);
}
__device__ inline double group16_max(double v) {
#pragma unroll
  for (int r = 8; r >= 1; r >>= 1)
    v = max_f64(v, __longlong_as_double((long long)row16_rotate((unsigned long long)__double_as_longlong(v), r)));
  return v;
}
__device__ inline double group16_min(double v) {
#pragma unroll
  for (int r = 8; r >= 1; r >>= 1)
    v = min_f64(v, __longlong_as_double((long long)row16_rotate((unsigned long long)__double_as_longlong(v), r)));
  return v;
}

// Lists the set bits of a front bitmap of at most blockDim.x words (LDS) in ascending order into perm[base ...].  A
// thread takes a word; when some word is dense (a front of neighbouring rows: 64 stores from one thread, one after
// the other, made a level of the listing slower than a level of the peeling) the words are instead taken by whole
// waves, a lane per bit.  word_base: nwords ints of LDS; scratch: 32 ints.  The barriers order LDS traffic only.
__device__ inline void list_front_words(const uint64_t* front_lds, int nwords, int* __restrict__ perm, int base,
                                        int* word_base, int* scratch) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, waves = blockDim.x >> 6;
  const uint64_t bits = tid < nwords ? front_lds[tid] : 0ull;
  const int mine = __popcll(bits);
  int incl = mine;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const int up = __shfl_up(incl, off);
    if (lane >= off) incl += up;
  }
  const int densest = wave_max(mine);
  if (lane == 63) {
    scratch[wave] = incl;
    scratch[16 + wave] = densest;
  }
  lds_barrier();
  int pos = base + incl - mine, heavy = 0;
  for (int v = 0; v < waves; ++v) {
    if (v < wave) pos += scratch[v];
    heavy = max(heavy, scratch[16 + v]);
  }
  if (heavy <= 12) {
    uint64_t left = bits;
    while (left) {
      perm[pos++] = tid * 64 + __ffsll((unsigned long long)left) - 1;
      left &= left - 1;
    }
  } else {
    if (tid < nwords) word_base[tid] = pos;
    lds_barrier();
    for (int w = wave; w < nwords; w += waves) {  // wave-uniform
      const uint64_t b = front_lds[w];
      if ((b >> lane) & 1ull) perm[word_base[w] + __popcll(b & ((1ull << lane) - 1ull))] = w * 64 + lane;
    }
  }
  lds_barrier();
}

// ---- The crowding distances and the order of a small last front, by the workgroups that have just peeled it.
// When the peeling stops, every sweeping workgroup holds the units of the last level in registers: the slots of
// the last front.  Ordering that front in a kernel of its own costs the launch (about 4.7 us on this device) and three
// chains of dependent loads (the control block, the listing, the costs); here the candidates get a number from the
// records (the same in every workgroup), their costs and original indices are fetched once, every workgroup works
// out the distances of its share (candidate e belongs to workgroup e mod sweepers; sixteen lanes scan all candidates
// for the two neighbours in every objective's order, see crowd_small_front in finish.hpp), publishes them as
// (distance key, original index) composites in a buffer that all workgroups poll -- a zero entry is one that has
// not arrived -- and places its candidates by counting the smaller composites.  Same results as the kernels of
// finish.hpp, except that the costs are read back from their order-preserving keys, under which -0.0 is +0.0 (the
// sign of a distance of zero can differ) and every NaN is the same NaN.
constexpr int kTailRows = 2048;        // candidates (four per thread in the poll of the buffer)
constexpr int kTailCopies = 8;         // of the buffer that every workgroup polls: one per die, like the records
constexpr int kTailValues = 4096;      // candidates x objectives: 12 bytes of LDS each
constexpr int kTailObjectives = 64;

__host__ __device__ inline bool peel_tail_applies(int64_t nv, int m) {
  return nv >= 1 && nv <= kTailRows && nv * m <= kTailValues && m <= kTailObjectives;
}
// Bytes of LDS that the tail needs at most for a population of n rows (0: it never applies).
__host__ inline size_t peel_tail_lds_bytes(int n, int m) {
  if (m > kTailObjectives) return 0;
  int64_t rows = n < kTailRows ? n : kTailRows;
  if (rows * m > kTailValues) rows = kTailValues / m;
  if (rows < 1) return 0;
  return (size_t)(12 * rows * m + 8 * rows + 16 * m + 8 * 256 + 64);
}

struct PeelTail {
  int mode;  // 0: ranks only; 2: crowding distances and selection order of the last front
  int m, npad;
  const float* xs_sorted;  // fitness by slot, structure of arrays, columns npad apart
  float* dist;             // by original index
  int* order;              // selection order
  unsigned long long* buffer;  // kTailCopies x kTailRows entries, zero at the start of the call
};

// Grid: 1 lister + `sweepers` sweeping workgroups of kLdsPeelThreads threads, all resident at once (every workgroup
// waits for every other one).  Dynamic LDS: lds_peel_bytes().  The matrix must be complete in `dom`; rank, the
// crowding-distance fill, the front sizes and listings and the control block are written as by count_kernel +
// peel_records_kernel.  Stops as soon as the fronts built so far hold stop_count rows.
template <bool MANY>  // several populations in the launch, one per blockIdx.z (the other instance is compiled without the pointer moves)
__global__ __launch_bounds__(kLdsPeelThreads) void peel_lds_kernel(
    const uint64_t* __restrict__ dom, int64_t wstride, int nwords, int n, const int* __restrict__ orig_of,
    int* __restrict__ rank, float* __restrict__ dist_fill, uint64_t* __restrict__ fronts_slot,
    uint64_t* __restrict__ fronts_orig, int* __restrict__ fsize, int* __restrict__ perm, int* __restrict__ fstart,
    Ctrl* __restrict__ ctrl, int stop_count, unsigned spin_limit, unsigned long long* __restrict__ records, int sweepers,
    PeelTail tail, int64_t ws_step) {
  extern __shared__ __attribute__((aligned(16))) uint64_t lds[];  // the rows are read 16 bytes at a time
  __shared__ int sh[48];
  if constexpr (MANY) {
    to_population(ws_step, dom, orig_of, rank, dist_fill, fronts_slot, fronts_orig, fsize, perm, fstart, ctrl, records);
    to_population(ws_step, tail.xs_sorted, tail.dist, tail.order, tail.buffer);
  }
  if (coherent_load(&ctrl->err) != 0) return;
  int units = 2;  // per record: the largest power of two up to 32 that gives every sweeper a record
  while (units * 2 * sweepers <= kRecUnits && units < 32) units *= 2;
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  constexpr int kWaves = kLdsPeelThreads / 64;
  using Rec = RecFormat<false>;

  if (blockIdx.x == 0) {
    // ---- lister: builds every front in original-index space from the records, lists it into perm (ascending
    // original index, which makes perm a stable ordering by rank) and recycles record slots and bitmaps
    // (the slot -> original index table sits in LDS: a look-up in memory per record would make a level of the
    // listing slower than a level of the peeling, and the kernel lasts as long as its slowest workgroup)
    uint64_t* front_lds = lds;
    int* word_base = reinterpret_cast<int*>(front_lds + nwords);
    uint16_t* orig_lds = reinterpret_cast<uint16_t*>(word_base + nwords);
    for (int j = tid; j < n; j += blockDim.x) orig_lds[j] = (uint16_t)orig_of[j];
    int ranked = 0;
    bool prev_overflow = false;
    // The two units that this thread reads are loaded a level ahead, before the listing of the present level: while
    // the lister is behind the sweepers they are there already, and a level costs no memory round trip.  The
    // barriers of the loop order LDS traffic only, so that they do not wait for that load.
    auto units_of = [&](int level) {
      return records + ((size_t)(level % kRecRing) * kRecCopies + kRecSweeperCopies) * kRecUnits;
    };
    const bool have = 2 * tid < sweepers * units;
    unsigned long long ahead[2] = {~0ull, ~0ull};
    if (have) {
      ahead[0] = coherent_load(units_of(0) + 2 * tid);
      ahead[1] = coherent_load(units_of(0) + 2 * tid + 1);
    }
    for (int level = 0;; ++level) {
      for (int w = tid; w < nwords; w += blockDim.x) front_lds[w] = 0ull;
      if (tid == 0) {
        sh[1] = 0;
        sh[2] = 0;
      }
      lds_barrier();
      unsigned long long v[2] = {ahead[0], ahead[1]};
      const unsigned gen = (unsigned)level + 1u;
      EVX_TRACE(level, 0);
      bool fine = true;
      if (have && ((unsigned)(v[0] >> 48) != (gen & 0xFFFFu) || (unsigned)(v[1] >> 48) != (gen & 0xFFFFu)))
        fine = poll_record_pair(units_of(level), sweepers * units, gen, v, nullptr, 0, &ctrl->err, spin_limit);
      // (the counts of the records are added up wave by wave: 255 atomics on one LDS word queue for a microsecond)
      int counted = 0;
      bool overflowed = false;
      if (fine) {
#pragma unroll
        for (int k = 0; k < 2; ++k) {
          if (2 * tid + k >= sweepers * units) continue;  // past the last record
          const int i = (2 * tid + k) & (units - 1);
          Rec::read(
              v[k], i == 0,
              [&](int count, bool overflow) {
                counted += count;
                overflowed |= overflow;
              },
              [&](int slot) {
                const int o = orig_lds[slot];
                atomicOr(reinterpret_cast<unsigned long long*>(&front_lds[o >> 6]), 1ull << (o & 63));
              });
        }
      }
      counted = wave_sum(counted);
      const bool any_overflow = __builtin_amdgcn_ballot_w64(overflowed) != 0ull;
      const bool any_failed = __builtin_amdgcn_ballot_w64(!fine) != 0ull;
      if (lane == 0) {
        if (counted) atomicAdd(&sh[1], counted);
        if (any_overflow || any_failed) atomicOr(&sh[2], (any_overflow ? 1 : 0) | (any_failed ? 2 : 0));
      }
      if (!fine) coherent_store(&ctrl->err, kErrBarrierTimeout);
      if (have) {
        ahead[0] = coherent_load(units_of(level + 1) + 2 * tid);
        ahead[1] = coherent_load(units_of(level + 1) + 2 * tid + 1);
      }
      EVX_TRACE(level, 1);
      lds_barrier();
      if (sh[2] & 2) return;
      const int size = sh[1];
      const bool overflow = (sh[2] & 1) != 0;
      const bool clearing = prev_overflow || level == 1;  // (buffer 0 may also hold the front 0 that count_kernel found)
      if (overflow) {
        const uint64_t* cur = fronts_orig + (int64_t)(level % kFrontBuffers) * nwords * kFrontStride;
        for (int w = tid; w < nwords; w += blockDim.x) front_lds[w] |= coherent_load(&cur[(int64_t)w * kFrontStride]);
      }
      if (clearing) {
        // every sweeper has published generation `level`, so it has finished with the bitmaps of front level-1
        uint64_t* prev_slot = fronts_slot + (int64_t)((level - 1) % kFrontBuffers) * nwords * kFrontStride;
        uint64_t* prev_orig = fronts_orig + (int64_t)((level - 1) % kFrontBuffers) * nwords * kFrontStride;
        for (int w = tid; w < nwords; w += blockDim.x) {
          coherent_store(&prev_slot[(int64_t)w * kFrontStride], (uint64_t)0);
          coherent_store(&prev_orig[(int64_t)w * kFrontStride], (uint64_t)0);
        }
      }
      prev_overflow = overflow;
      if (clearing)
        __syncthreads();  // waits for the clearing stores of this block's waves
      else
        lds_barrier();
      if (tid == 0) coherent_store(&ctrl->listed, level);  // records <= level consumed, bitmaps < level cleared
      const bool last = size <= 0 || ranked + size >= stop_count;
      EVX_TRACE(level, 2);
      if (perm) list_front_words(front_lds, nwords, perm, ranked, word_base, sh + 8);
      EVX_TRACE(level, 3);
      if (tid == 0) {
        fstart[level] = ranked;
        fsize[level] = size;
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
      lds_barrier();
    }
  }

  // ---- sweepers
  const int sb = (int)blockIdx.x - 1;
  const int row_step = sweepers * kWaves;
  const int per_wave = (n + row_step - 1) / row_step;  // <= kLdsPeelRowsPerWave (the host has checked)
  const int rows_cap = per_wave * kWaves;
  uint64_t* alive_lds = lds;
  int* row_off = reinterpret_cast<int*>(alive_lds + nwords);
  int* found = row_off + ((rows_cap + 4) & ~3);
  uint64_t* rows_lds = reinterpret_cast<uint64_t*>(found + 2 * rows_cap);
  // the block's rows in LDS, wave by wave: entry t = wave * per_wave + k is the k-th row of that wave
  const int first_row = sb * kWaves + wave;
  EVX_TRACE(62, 0);
  // lane k owns the wave's k-th row
  const int64_t my_slot = first_row + (int64_t)lane * row_step;
  const bool have_row = lane < per_wave && my_slot < n;
  const int st_orig = have_row ? orig_of[my_slot] : 0;
  {
    // exclusive scan of the row lengths (rows_cap <= blockDim.x)
    const int64_t jt = tid < rows_cap ? (int64_t)sb * kWaves + tid / per_wave + (int64_t)(tid % per_wave) * row_step : n;
    const int rw = jt < n ? row_words((int)jt) : 0;
    int incl = rw;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const int up = __shfl_up(incl, off);
      if (lane >= off) incl += up;
    }
    if (lane == 63) sh[8 + wave] = incl;
    if (tid < 8) sh[tid] = 0;
    __syncthreads();
    int before = 0;
    for (int v = 0; v < wave; ++v) before += sh[8 + v];
    if (tid < rows_cap) row_off[tid] = before + incl - rw;
    if (tid == rows_cap - 1) row_off[rows_cap] = before + incl;
  }
  for (int w = tid; w < nwords; w += blockDim.x) {
    const int lo = w * 64;
    alive_lds[w] = lo + 64 <= n ? ~0ull : (lo >= n ? 0ull : ((1ull << (n - lo)) - 1ull));
  }
  __syncthreads();

  EVX_TRACE(62, 1);
  // ---- copy this wave's rows into LDS.  The rows of a wave are one run of 16-byte pieces in LDS; the lanes take
  // the pieces in turn, eight loads in flight each, whatever the lengths of the rows (a wave's first rows are
  // short: row by row most lanes would idle, and the copy costs one memory round trip per group of rows)
  {
    const int* my_off = row_off + wave * per_wave;
    const int piece0 = my_off[0] >> 1, piece_end = my_off[per_wave] >> 1;  // rows past n have no pieces
    int k = 0, k_end = my_off[1] >> 1;  // the row that holds the lane's present piece ends before piece k_end
    for (int p0 = piece0 + lane; p0 - lane < piece_end; p0 += 16 * 64) {
      // where the lane's next sixteen pieces come from (words from the start of the matrix; a piece past the end
      // reads the first piece of the matrix and is dropped), then all loads, then all stores
      int from[16];
#pragma unroll
      for (int u = 0; u < 16; ++u) {
        const int p = p0 + u * 64;
        from[u] = 0;
        if (p < piece_end) {
          while (p >= k_end) {
            ++k;
            k_end = my_off[k + 1] >> 1;
          }
          from[u] = (int)((first_row + (int64_t)k * row_step) * wstride) + (2 * p - my_off[k]);
        }
      }
      ulonglong2 v[16];
#pragma unroll
      for (int u = 0; u < 16; ++u) v[u] = *reinterpret_cast<const ulonglong2*>(dom + from[u]);
#pragma unroll
      for (int u = 0; u < 16; ++u) {
        const int p = p0 + u * 64;
        if (p < piece_end) *reinterpret_cast<ulonglong2*>(rows_lds + 2 * p) = v[u];
      }
    }
  }
  EVX_TRACE(62, 2);
  // the witness of every row: its highest non-empty word (the lanes of a wave see their own LDS writes in order)
  // Every lane walks down its own row, eight words a step, all rows of the wave side by side (the wave as a whole
  // on one row after the other cost 2 us here at 20 000 rows: a row's highest dominator lies a few dozen words
  // below its own slot, rows of similar key sums rarely dominate one another).
  int st_word = -1, st_off = 0;
  uint64_t st_bits = 0ull;
  const int my_words = have_row ? row_words((int)my_slot) : 0;
  if (have_row) st_off = row_off[wave * per_wave + lane];
  // (no row is ranked yet, so every bit counts; a row is a whole number of 16-byte pieces, read as such; the words
  // of a step are ORed together first: a row without dominators -- every row of a converged population -- is walked
  // to its end, at a third of the instructions that looking at every word would take)
  for (int top = my_words - 1; __builtin_amdgcn_ballot_w64(st_word < 0 && top >= 0) != 0ull; top -= 16) {
    ulonglong2 v[8];
    uint64_t any = 0ull;
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      const int w = top - 1 - 2 * q;  // the piece holds words w and w + 1
      const bool in = st_word < 0 && w >= 0;
      v[q] = in ? *reinterpret_cast<const ulonglong2*>(rows_lds + st_off + w) : make_ulonglong2(0ull, 0ull);
      any |= v[q].x | v[q].y;
    }
    if (__builtin_amdgcn_ballot_w64(any != 0ull) != 0ull) {
#pragma unroll
      for (int q = 7; q >= 0; --q) {
        const int w = top - 1 - 2 * q;
        if (v[q].x != 0ull) {
          st_word = w;
          st_bits = v[q].x;
        }
        if (v[q].y != 0ull) {
          st_word = w + 1;
          st_bits = v[q].y;
        }
      }
    }
  }
  if (have_row && st_word < 0) {  // no dominator: front 0
    const int e = atomicAdd(&sh[0], 1);
    found[2 * e] = (int)my_slot;
    found[2 * e + 1] = st_orig;
  }
  if (have_row) {
    rank[st_orig] = st_word < 0 ? 0 : kRankUnset;
    // (written through: the distance of a row of the last front is stored again at the end of this kernel by
    // another workgroup, maybe on another die, whose store must not be overtaken by this one's write-back)
    if (dist_fill) coherent_store(&dist_fill[st_orig], -INFINITY);
  }
  EVX_TRACE(62, 3);

  // The counters of a level live in sh[4 p .. 4 p + 3], p = the parity of the level: [0] rows this block ranks,
  // [1] rows all blocks rank, [2] bit 0: some block overflowed its record, bit 1: give up.  Those of the next level
  // are cleared in the middle of this one (between two barriers that the level needs anyway).
  int level = 0;
  int ranked = 0;  // rows in fronts 0 .. level-1
  for (;;) {
    int* const cnts = sh + 4 * (level & 1);
    int* const next_cnts = sh + 4 * ((level + 1) & 1);
    EVX_TRACE(level, 0);
    lds_barrier();  // the list of the rows of front `level` found by this block is complete
    const int cnt = cnts[0];
    if (tid < 4) next_cnts[tid] = 0;
    const unsigned gen = (unsigned)level + 1u;
    unsigned long long* gen_units = records + (size_t)(level % kRecRing) * kRecCopies * kRecUnits;
    // thread t writes unit t % units of the record into copy t / units
    unsigned long long* mine = gen_units + (size_t)(tid / units) * kRecUnits + (size_t)sb * units + (tid % units);
    if (cnt <= Rec::capacity(units)) {
      if (tid < units * kRecCopies) coherent_store(mine, Rec::unit_for(gen, tid % units, found, cnt, false));
    } else {
      uint64_t* next_slot = fronts_slot + (int64_t)(level % kFrontBuffers) * nwords * kFrontStride;
      uint64_t* next_orig = fronts_orig + (int64_t)(level % kFrontBuffers) * nwords * kFrontStride;
      for (int e = tid; e < cnt; e += blockDim.x) {
        const int slot = found[2 * e], orig = found[2 * e + 1];
        atomicOr(reinterpret_cast<unsigned long long*>(next_slot + (int64_t)(slot >> 6) * kFrontStride), 1ull << (slot & 63));
        atomicOr(reinterpret_cast<unsigned long long*>(next_orig + (int64_t)(orig >> 6) * kFrontStride), 1ull << (orig & 63));
      }
      __syncthreads();  // every wave has waited for its own atomics
      if (tid < units * kRecCopies) coherent_store(mine, Rec::unit_for(gen, tid % units, found, cnt, true));
    }
    // the records of everybody: barrier and front exchange in one.  Thread 0 also makes sure that the lister has
    // recycled what generation level + 2 will overwrite.
    EVX_TRACE(level, 1);
    unsigned long long v[2];
    const bool fine = poll_record_pair(gen_units + (size_t)(blockIdx.x % kRecSweeperCopies) * kRecUnits, sweepers * units, gen, v,
                                       tid == 0 ? &ctrl->listed : nullptr, level + 2 - kRecRing, &ctrl->err, spin_limit);
    EVX_TRACE(level, 2);
    // (every record's count is added up wave by wave first: 255 atomics on one LDS word would queue for more than
    // a microsecond)
    int counted = 0;
    bool overflowed = false;
    if (fine) {
#pragma unroll
      for (int k = 0; k < 2; ++k) {
        if (2 * tid + k >= sweepers * units) continue;  // past the last record
        const int i = (2 * tid + k) & (units - 1);
        Rec::read(
            v[k], i == 0,
            [&](int count, bool overflow) {
              counted += count;
              overflowed |= overflow;
            },
            [&](int slot) { atomicAnd(reinterpret_cast<unsigned long long*>(&alive_lds[slot >> 6]), ~(1ull << (slot & 63))); });
      }
    }
    counted = wave_sum(counted);
    const bool any_overflow = __builtin_amdgcn_ballot_w64(overflowed) != 0ull;
    const bool any_failed = __builtin_amdgcn_ballot_w64(!fine) != 0ull;
    if (lane == 0) {
      if (counted) atomicAdd(&cnts[1], counted);
      if (any_overflow || any_failed) atomicOr(&cnts[2], (any_overflow ? 1 : 0) | (any_failed ? 2 : 0));
    }
    if (!fine) coherent_store(&ctrl->err, kErrBarrierTimeout);
    lds_barrier();  // the bitmap of unranked rows and the counters of the level are complete
    EVX_TRACE(level, 3);
    const int flags = cnts[2];
    const int size = cnts[1];
    if (flags & 2) break;
    if (flags & 1) {  // the same in every thread
      const uint64_t* cur = fronts_slot + (int64_t)(level % kFrontBuffers) * nwords * kFrontStride;
      for (int w = tid; w < nwords; w += blockDim.x) alive_lds[w] &= ~coherent_load(&cur[(int64_t)w * kFrontStride]);
      lds_barrier();
    }
    if (size <= 0 || ranked + size >= stop_count) {
      // front `level` is the last one: a small one is ordered right here (the overflow path leaves no slots in v)
      if (tail.mode == 2 && (flags & 1) == 0 && peel_tail_applies(size, tail.m)) {
        const int nv = size, start = ranked, want = stop_count - ranked, m = tail.m;
        // Composites (key << 15 | original index: at most 47 bits, the population has at most 32 768 rows) are held
        // as doubles, which represent them exactly: the vector unit compares doubles and takes their maximum at the
        // rate of 32-bit values, 64-bit integers at a quarter of it, and the scans below are nothing but comparisons.
        double* comp = reinterpret_cast<double*>(lds);       // [m][nv], then the distance composites
        double* ends = comp + (size_t)nv * m;                // [m][2]
        int* t_slot = reinterpret_cast<int*>(ends + 2 * m);  // [nv]
        int* t_orig = t_slot + nv;                                               // [nv]
        int* rec_cnt = t_orig + nv;                                              // [256] rows per record, then their prefix
        EVX_TRACE(61, 0);
        lds_barrier();  // nobody reads the bitmap or the rows any more
        // number the candidates: record by record, in the order of the record's slots
        const int n_rec = sweepers;
#pragma unroll
        for (int k = 0; k < 2; ++k) {
          const int u = 2 * tid + k;
          if (u < sweepers * units && (u & (units - 1)) == 0)
            rec_cnt[u / units] = (int)((uint32_t)(v[k] >> (Rec::kBits * (Rec::kFields - 1))) & Rec::kMask & ~Rec::kOverflow);
        }
        lds_barrier();
        if (wave == 0) {  // exclusive prefix over at most 255 records: four per lane
          int c[4], sum = 0;
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            c[q] = 4 * lane + q < n_rec ? rec_cnt[4 * lane + q] : 0;
            sum += c[q];
          }
          int incl = sum;
#pragma unroll
          for (int off = 1; off < 64; off <<= 1) {
            const int up = __shfl_up(incl, off);
            if (lane >= off) incl += up;
          }
          int run = incl - sum;
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            if (4 * lane + q < n_rec) rec_cnt[4 * lane + q] = run;
            run += c[q];
          }
        }
        lds_barrier();
#pragma unroll
        for (int k = 0; k < 2; ++k) {
          const int u = 2 * tid + k;
          if (u >= sweepers * units) continue;
          const int b = u / units, i = u & (units - 1);
          // unit 0 carries the count and the record's first kFields - 1 slots, unit i the slots from kFields * i - 1 on
#pragma unroll
          for (int fld = 0; fld < Rec::kFields; ++fld) {
            if (i == 0 && fld == 0) continue;
            const uint32_t field = (uint32_t)(v[k] >> (Rec::kBits * (Rec::kFields - 1 - fld))) & Rec::kMask;
            if (field != Rec::kNil) t_slot[rec_cnt[b] + (i == 0 ? fld - 1 : Rec::kFields * i - 1 + fld)] = (int)field;
          }
        }
        lds_barrier();
        // (cost key, original index) of every candidate in every objective: one round trip to memory (at most
        // kTailValues = 8 * 512 items: a thread's eight pairs of loads are all in flight together)
        {
          constexpr int kPerThread = kTailValues / kLdsPeelThreads;
          int orig_v[kPerThread];
          float cost_v[kPerThread];
#pragma unroll
          for (int q = 0; q < kPerThread; ++q) {
            const int idx = tid + q * kLdsPeelThreads;
            const int idc = idx < nv * m ? idx : 0;
            const int k = idc / nv, e = idc - k * nv;
            const int slot = t_slot[e];
            orig_v[q] = orig_of[slot];
            cost_v[q] = tail.xs_sorted[(int64_t)k * tail.npad + slot];
          }
#pragma unroll
          for (int q = 0; q < kPerThread; ++q) {
            const int idx = tid + q * kLdsPeelThreads;
            if (idx < nv * m) {
              comp[idx] = tail_composite(ordered_key(cost_v[q]), orig_v[q]);
              if (idx < nv) t_orig[idx] = orig_v[q];
            }
          }
        }
        lds_barrier();
        EVX_TRACE(61, 1);
        for (int k = wave; k < m; k += kWaves) {  // first and last composite of every objective
          double lo = INFINITY, hi = -1.0;
          for (int e = lane; e < nv; e += 64) {
            const double c = comp[k * nv + e];
            lo = min_f64(lo, c);
            hi = max_f64(hi, c);
          }
          lo = group16_min(lo);  // (rotations inside rows of sixteen lanes cost a tenth of a permute through LDS)
          hi = group16_max(hi);
#pragma unroll
          for (int off = 16; off < 64; off <<= 1) {
            lo = min_f64(lo, shfl_xor_f64(lo, off));
            hi = max_f64(hi, shfl_xor_f64(hi, off));
          }
          if (lane == 0) {
            ends[2 * k] = lo;
            ends[2 * k + 1] = hi;
          }
        }
        lds_barrier();
        EVX_TRACE(59, 0);
        // this workgroup's candidates are e = sb, sb + sweepers, ...; a group of lanes takes one (candidate,
        // objective) pair, so that the objectives of a candidate are scanned side by side, and leaves the term of
        // the distance (NaN bit pattern 0xFFFFFFFF for "first or last of the objective") in LDS.  A group is sixteen
        // lanes, or 32 or 64 when the workgroup has so few pairs that most of its lanes would have nothing to do.
        const int mine_n = sb < nv ? (nv - 1 - sb) / sweepers + 1 : 0;
        const int gl = tail_group_lanes(mine_n * m);
        const int sub = tid & (gl - 1);
        const int groups = kLdsPeelThreads / gl;
        float* term_lds = reinterpret_cast<float*>(rec_cnt + 256);  // [candidates of this workgroup][m]
        constexpr uint32_t kBoundaryTerm = 0xFFFFFFFFu;
        for (int it = tid / gl; it < mine_n * m; it += groups) {  // (whole groups leave the loop together)
          const int j = it / m, k = it - j * m;
          const int e = sb + j * sweepers;
          const double* row = comp + (size_t)k * nv;
          const double mine = row[e];
          double below = -1.0, above = INFINITY;  // no composite is negative or infinite
          for (int p0 = sub; p0 < nv; p0 += 8 * gl) {  // eight partners per step, their LDS reads in flight together
            double c[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) c[u] = p0 + gl * u < nv ? row[p0 + gl * u] : mine;
#pragma unroll
            for (int u = 0; u < 8; ++u) {
              below = max_f64(below, c[u] < mine ? c[u] : -1.0);
              above = min_f64(above, c[u] > mine ? c[u] : INFINITY);
            }
          }
          below = group16_max(below);
          above = group16_min(above);
          for (int off = 16; off < gl; off <<= 1) {
            below = max_f64(below, shfl_xor_f64(below, off));
            above = min_f64(above, shfl_xor_f64(above, off));
          }
          if (sub == 0) {
            float term = __uint_as_float(kBoundaryTerm);  // first or last of this objective (non_dominate.py:226-227)
            if (below >= 0.0 && above != INFINITY) {
              const float span = cost_of_key(tail_composite_key(ends[2 * k + 1])) - cost_of_key(tail_composite_key(ends[2 * k]));
              term = (cost_of_key(tail_composite_key(above)) - cost_of_key(tail_composite_key(below))) / span;
            }
            term_lds[it] = term;
          }
        }
        lds_barrier();
        EVX_TRACE(59, 1);
        for (int j = tid; j < mine_n; j += blockDim.x) {
          const int e = sb + j * sweepers;
          bool boundary = false;
          float acc = 0.0f;
          for (int k = 0; k < m; ++k) {
            const float term = term_lds[j * m + k];
            if (__float_as_uint(term) == kBoundaryTerm)
              boundary = true;
            else
              acc = k == 0 ? term : acc + term;
          }
          const float d = boundary ? INFINITY : acc;
          coherent_store(&tail.dist[t_orig[e]], d);
          const unsigned long long entry = ((unsigned long long)ordered_key(-d) << 32) | (unsigned)t_orig[e];
#pragma unroll
          for (int c = 0; c < kTailCopies; ++c) coherent_store(&tail.buffer[c * kTailRows + e], entry);
        }
        EVX_TRACE(61, 2);
        lds_barrier();  // the composites of the objectives are no longer needed
        // everybody's distance composites: entries 4 t .. 4 t + 3 are this thread's
        {
          typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
          const int e0 = 4 * tid;
          bool pending0 = e0 < nv, pending1 = e0 + 2 < nv, fine_poll = true;
          // (both loads of a round are in flight together; the buffer holds kTailRows entries, a multiple of four,
          // so the second load of a thread whose first is in range stays inside it)
          WaitBound bound(spin_limit);
          for (unsigned spins = 0; pending0 || pending1; ++spins) {
            u32x4 r0, r1;
            asm volatile("global_load_dwordx4 %0, %2, off sc1\n\tglobal_load_dwordx4 %1, %2, off offset:16 sc1\n\ts_waitcnt vmcnt(0)"
                         : "=&v"(r0), "=&v"(r1)
                         : "v"(tail.buffer + (blockIdx.x % kTailCopies) * kTailRows + e0)
                         : "memory");
            if (pending0) {
              const unsigned long long a = ((unsigned long long)r0.y << 32) | r0.x, b = ((unsigned long long)r0.w << 32) | r0.z;
              if (a != 0ull && (e0 + 1 >= nv || b != 0ull)) {
                comp[e0] = tail_composite((uint32_t)(a >> 32), (int)(uint32_t)a);
                if (e0 + 1 < nv) comp[e0 + 1] = tail_composite((uint32_t)(b >> 32), (int)(uint32_t)b);
                pending0 = false;
              }
            }
            if (pending1) {
              const unsigned long long a = ((unsigned long long)r1.y << 32) | r1.x, b = ((unsigned long long)r1.w << 32) | r1.z;
              if (a != 0ull && (e0 + 3 >= nv || b != 0ull)) {
                comp[e0 + 2] = tail_composite((uint32_t)(a >> 32), (int)(uint32_t)a);
                if (e0 + 3 < nv) comp[e0 + 3] = tail_composite((uint32_t)(b >> 32), (int)(uint32_t)b);
                pending1 = false;
              }
            }
            if (bound.expired(spins) || ((spins & 63u) == 63u && coherent_load(&ctrl->err) != 0)) {
              fine_poll = false;
              break;
            }
          }
          if (!fine_poll) {
            coherent_store(&ctrl->err, kErrBarrierTimeout);
            next_cnts[3] = 1;  // (cleared with the counters of the level that will not come)
          }
        }
        EVX_TRACE(61, 3);
        lds_barrier();
        if (next_cnts[3] == 0) {  // every entry has arrived (a wait that gave up, here or elsewhere, ended the polls)
          const int gc = tail_group_lanes(mine_n), sub_c = tid & (gc - 1);
          for (int j = tid / gc; j < mine_n; j += kLdsPeelThreads / gc) {
            const int e = sb + j * sweepers;
            const double mine = comp[e];
            int smaller = 0;
            for (int p0 = sub_c; p0 < nv; p0 += 8 * gc) {
              double c[8];
#pragma unroll
              for (int u = 0; u < 8; ++u) c[u] = p0 + gc * u < nv ? comp[p0 + gc * u] : INFINITY;
#pragma unroll
              for (int u = 0; u < 8; ++u) smaller += c[u] < mine;
            }
            smaller = group16_sum(smaller);
            for (int off = 16; off < gc; off <<= 1) smaller += __shfl_xor(smaller, off);
            if (sub_c == 0 && smaller < want) tail.order[start + smaller] = t_orig[e];
          }
          if (sb == 0 && tid == 0) ctrl->tail_done = 1;
          EVX_TRACE(60, 0);
        }
      }
      break;
    }
    ranked += size;
    ++level;  // now building front `level`
    int* const build = sh + 4 * (level & 1);
    const bool need = st_word >= 0 && (st_bits & alive_lds[st_word < 0 ? 0 : st_word]) == 0ull;
    uint64_t todo = __builtin_amdgcn_ballot_w64(need);
    while (todo) {
      const int l = __ffsll((unsigned long long)todo) - 1;
      todo &= todo - 1;
      const int off = __builtin_amdgcn_readlane(st_off, l);
      const int nw = __builtin_amdgcn_readlane(st_word, l);  // words from the dead witness upwards hold no unranked dominator
      int word;
      uint64_t bits;
      lds_row_highest(rows_lds + off, nw, alive_lds, word, bits);
      if (lane == l) {
        st_word = word;
        st_bits = bits;
        if (word < 0) {
          rank[st_orig] = level;
          const int e = atomicAdd(&build[0], 1);
          found[2 * e] = first_row + l * row_step;
          found[2 * e + 1] = st_orig;
        }
      }
    }
  }
}

}  // namespace evx
