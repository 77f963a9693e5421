// Pairwise Pareto dominance -> bit matrix.
//
// Reference semantics (src/evox/operators/selection/non_dominate.py:6-26):
//   A[i, j] = all_k(x[i,k] <= x[j,k]) and any_k(x[i,k] < x[j,k])      (any NaN makes the pair False)
//
// Layout produced here ("dominated-by" rows): dom[j * wstride + w] holds, in bit b, A[64*w + b, j].
// Row j therefore lists the dominators of j; its popcount is the domination count of
// non_dominate.py:188 and one peel pass is popcount(row & front) (non_dominate.py:29-59).
// Rows and columns are SLOTS: the population relabelled by ascending row key (order.hpp), which makes
// the matrix strictly lower triangular; word pairs that lie wholly above the diagonal are neither
// evaluated nor stored, and no reader looks at them (row j is defined up to word 2 * (j / 128) + 1).
//
// Work split: lane = j (fitness of 64 rows held in VGPRs), loop over i with x[i, :] fetched by
// scalar loads (the index is wave-uniform), so every `<=` is one v_cmp_le_f32 with an SGPR operand
// whose result is a 64-lane mask in an SGPR pair; the per-objective masks are ANDed on the scalar
// unit.  "any strictly less" is replaced by one integer compare: with key(i) = sum_k w_k ordered_key(x[i,k]) (positive weights w_k, key_weight below)
// and all_k(x[i,k] <= x[j,k]) already true (which rules out NaN on both sides), the rows differ in
// some objective exactly when key(i) != key(j), because the per-objective keys are ordered the same
// way as the floats and sum without overflow.  The compare is made on a 32-bit stand-in for the key,
// kid(slot) = first slot that holds the same key (equal ids <=> equal keys), which halves the scalar
// bytes per dominator and is one full-rate v_cmp_ne_u32.  The lane mask is then shifted into the lane's own
// 32-bit accumulator with v_addc_co_u32 (acc = acc + acc + carry), which performs the transpose from
// "mask over j" to "word over i" at one VALU instruction per 64 pairs.
//
// Faster still when every value is finite (the usual case; the slot sort reports it): the test is done in
// VGPR arithmetic, which this hardware issues at twice the rate of compares that write a lane mask.
// With d_k = x[j,k] - x[i,k] (exact in sign, zero only for equal values once -0.0 is stored as +0.0; an
// overflow to infinity keeps the sign), i dominates j exactly when no d_k is negative and some d_k is not
// zero, i.e. when the bitwise OR of the d_k, read as a signed integer, is positive: M v_sub_f32 with a
// scalar operand, (M-1)/2 v_or3_b32, one v_med3_i32 (clamp to 0..1) and one v_lshl_or_b32 into the lane's
// accumulator -- 6 full-rate instructions for M = 3 instead of 5 half-rate ones and 3 scalar ANDs
// (measured in a bare loop: 8.6 against 5.9 T pairs/s).  Up to three objectives one instruction fewer: the
// sign bit of the OR (some d_k negative: i is worse somewhere) goes into the accumulator by one v_alignbit_b32,
// the finished 32 bits are complemented, and the rows equal to j -- the only rows that are no worse anywhere and
// yet do not dominate -- are cleared as the slots from kid(j) on.  NaN and infinities would break the sign
// argument (inf - inf), so populations that hold any keep the compare form.
#pragma once

#include "common.hpp"
#include "order.hpp"

namespace evx {

// The row key of the bucket sort weighs the objectives slightly differently (16, 17, ..., 23, 16, ...).  Any positive
// weights keep what the key is for -- a dominator's key is strictly smaller, rows equal in every objective have equal
// keys -- and unequal ones keep the keys of a population that lies on a plane sum_k x[i,k] = const (normalised
// objectives, a converged front) apart: the integer image of a float is linear in the float within a binade, so
// with equal weights all rows whose values share their binades would get the same key, thousands of rows in one
// bucket (weights whose odd parts differ never cancel against the binades' powers of two).  Nearly equal, because the
// peel counts on rows of large key lying in deep fronts (weights 3, 5, 7 cost it 2 us at 20 000 x 3, weights 4, 5, 6 one).  At most
// 23 * 65535 * 2^32 < 2^53: no overflow.
__host__ __device__ inline uint32_t key_weight(int k) { return 16u + (uint32_t)(k & 7); }

// One kernel turns the caller's strided (n, m) fitness into structure-of-arrays form in original
// order (padded with NaN to npad, a multiple of 128 rows) plus the 64-bit row keys, leaves the
// (min, max) key of each block in `partials` for the slot sort, and clears the state arrays that
// later kernels accumulate into.  The third partial of a block says whether it met a NaN or an infinity.
// The population may come in two parts (rows 0..n_first-1 from f, the rest from f2: parents and
// offspring that the caller never concatenates, src/evox/algorithms/mo/nsga2.py:99-100).
// MANY: several populations in the launch, one per blockIdx.z (the instance for one population is compiled without
// the pointer moves).
template <bool MANY>
__global__ __launch_bounds__(256) void prepare_kernel(const float* __restrict__ f, int64_t stride_row, int64_t stride_col,
                                                      int n_first, const float* __restrict__ f2, int64_t stride_row2,
                                                      int64_t stride_col2, int n, int m, int npad, float* __restrict__ xs,
                                                      uint64_t* __restrict__ key, unsigned long long* __restrict__ partials,
                                                      uint32_t* __restrict__ zero_words, int64_t n_zero_words, int lexicographic,
                                                      int64_t f_step, int64_t f2_step, int64_t ws_step) {
  __shared__ unsigned long long red[2][4];
  __shared__ int any_bad;
  if constexpr (MANY) {  // the fitness of population b lies f_step elements behind that of population 0
    f += (int64_t)blockIdx.z * f_step;
    f2 += (int64_t)blockIdx.z * f2_step;
    to_population(ws_step, xs, key, partials, zero_words);
  }
  if (threadIdx.x == 0) any_bad = 0;
  __syncthreads();
  bool bad = false;
  const int64_t tid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t nthreads = (int64_t)gridDim.x * blockDim.x;
  unsigned long long lo = ~0ull, hi = 0ull;
  for (int64_t i = tid; i < npad; i += nthreads) {
    uint64_t s = 0;
    for (int k = 0; k < m; ++k) {
      const float v = i < n_first ? f[i * stride_row + k * stride_col]
                      : i < n     ? f2[(i - n_first) * stride_row2 + k * stride_col2]
                                  : __uint_as_float(0x7FC00000u);
      xs[(int64_t)k * npad + i] = v;
      // (two objectives ranked without a matrix, two.hpp: the rows in the order of the first objective, then the second)
      s = lexicographic ? (s << 32) | ordered_key(v) : s + (uint64_t)key_weight(k) * ordered_key(v);
      bad |= i < n && !(fabsf(v) <= 3.4028234663852886e38f);  // NaN or infinite
    }
    key[i] = s;
    if (i < n) {
      lo = s < lo ? s : lo;
      hi = s > hi ? s : hi;
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const unsigned long long a = __shfl_xor(lo, off), b = __shfl_xor(hi, off);
    lo = a < lo ? a : lo;
    hi = b > hi ? b : hi;
  }
  if ((threadIdx.x & 63) == 0) {
    red[0][threadIdx.x >> 6] = lo;
    red[1][threadIdx.x >> 6] = hi;
  }
  if (bad) any_bad = 1;
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int v = 1; v < 4; ++v) {
      lo = red[0][v] < lo ? red[0][v] : lo;
      hi = red[1][v] > hi ? red[1][v] : hi;
    }
    partials[3 * blockIdx.x] = lo;      // a block without rows leaves (all-ones, 0, 0): neutral
    partials[3 * blockIdx.x + 1] = hi;
    partials[3 * blockIdx.x + 2] = (unsigned long long)any_bad;
  }
  for (int64_t i = tid; i < n_zero_words; i += nthreads) zero_words[i] = 0u;
}

// Populations of at most kSmallSortRows rows: prepare_kernel and the four kernels of the bucket sort in one
// launch, with no dependence between workgroups.  Every workgroup computes the keys of all rows into LDS as
// composites (key << 12 | original index; keys are below 2^40 and indices below 2^12), then places its own
// sixteen rows by counting: the count of a row is split over the four quarters of a wave's lanes and the
// sixteen waves, each part counting over a sixty-fourth of the composites, and the first wave adds the
// shares up (a few thousand rows thus spread over the whole device: 10 against 20 us at 4096 x 3, 7 against
// 19 us at 2000 x 2).  slot = number of smaller
// composites, kid = number of smaller keys = first slot that holds the key; the outputs are those of
// prepare_kernel (xs, the state cleared) and of bucket_place_kernel (slot-ordered arrays, NaN / all-ones / -1
// padding up to npad), and the flag that says whether a NaN or an infinity was met.
constexpr int kSmallSortRows = 4096;
constexpr int kSmallSortValues = 28672;  // and at most this many fitness values (every workgroup reads all of them:
                                         // measured 14.8 against 21.3 us at 4096 x 7, 22.7 against 21.8 us at 4096 x 8)
constexpr int kSmallSortObjectives = 256;  // keys stay below 2^40, composites below 2^52: exact as doubles
constexpr int kSmallSortThreads = 1024;
constexpr int kSmallSortGroup = 16;  // rows placed by one workgroup

template <bool MANY>
__global__ __launch_bounds__(kSmallSortThreads) void small_sort_kernel(
    const float* __restrict__ f, int64_t stride_row, int64_t stride_col, int n_first, const float* __restrict__ f2,
    int64_t stride_row2, int64_t stride_col2, int n, int m, int npad, float* __restrict__ xs, SortParam* __restrict__ param_out,
    uint64_t* __restrict__ key_sorted, uint32_t* __restrict__ kid_sorted, float* __restrict__ xs_sorted, int* __restrict__ orig_of,
    uint32_t* __restrict__ zero_words, int64_t n_zero_words, int64_t f_step, int64_t f2_step, int64_t ws_step) {
  if constexpr (MANY) {
    f += (int64_t)blockIdx.z * f_step;
    f2 += (int64_t)blockIdx.z * f2_step;
    to_population(ws_step, xs, param_out, key_sorted, kid_sorted, xs_sorted, orig_of, zero_words);
  }
  // npad composites, held as doubles (they are below 2^47, so exact): the hardware compares doubles at the
  // rate of 32-bit values, 64-bit integers several times slower; +inf for the padding rows
  extern __shared__ double comp[];
  __shared__ int share[2][16 * (64 / kSmallSortGroup)][kSmallSortGroup];
  const int lane = threadIdx.x & 63, part = threadIdx.x >> 6;
  auto value = [&](int i, int k) {
    return i < n_first ? f[(int64_t)i * stride_row + k * stride_col] : f2[(int64_t)(i - n_first) * stride_row2 + k * stride_col2];
  };
  bool bad = false;
  {
    // every row of the population, kRowsPerThread per thread; the loads of one objective for all of a thread's
    // rows are independent and in flight together (a load per row and round trip would cost a memory latency
    // per 1024 rows)
    constexpr int kRowsPerThread = (kSmallSortRows + 127) / kSmallSortThreads + 1;
    uint64_t sum[kRowsPerThread];
#pragma unroll
    for (int t = 0; t < kRowsPerThread; ++t) sum[t] = 0;
    // rows of m consecutive floats are read four values at a time (the compiler merges them into one 16-byte
    // load per lane: with a separate load per objective every lane would use 4 bytes of each 32-byte sector)
    const bool packed = stride_col == 1 && stride_row == m && stride_col2 == 1 && stride_row2 == m;
    int k0 = 0;
    if (packed) {
      for (; k0 + 4 <= m; k0 += 4) {
        float v[kRowsPerThread][4];
#pragma unroll
        for (int t = 0; t < kRowsPerThread; ++t) {
          const int i = (int)threadIdx.x + t * kSmallSortThreads;
          const float* __restrict__ p = i < n_first ? f + (int64_t)i * m + k0 : f2 + (int64_t)(i - n_first) * m + k0;
#pragma unroll
          for (int u = 0; u < 4; ++u) v[t][u] = i < n ? p[u] : 0.0f;
        }
#pragma unroll
        for (int t = 0; t < kRowsPerThread; ++t)
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            sum[t] += ordered_key(v[t][u]);
            bad |= !(fabsf(v[t][u]) <= 3.4028234663852886e38f);  // NaN or infinite
          }
      }
    }
    for (int k = k0; k < m; ++k) {
      float v[kRowsPerThread];
#pragma unroll
      for (int t = 0; t < kRowsPerThread; ++t) {
        const int i = (int)threadIdx.x + t * kSmallSortThreads;
        v[t] = i < n ? value(i, k) : 0.0f;
      }
#pragma unroll
      for (int t = 0; t < kRowsPerThread; ++t) {
        sum[t] += ordered_key(v[t]);
        bad |= !(fabsf(v[t]) <= 3.4028234663852886e38f);  // NaN or infinite
      }
    }
#pragma unroll
    for (int t = 0; t < kRowsPerThread; ++t) {
      const int i = (int)threadIdx.x + t * kSmallSortThreads;
      if (i < npad) comp[i] = i < n ? (double)((sum[t] << 12) | (uint64_t)i) : (double)INFINITY;
    }
  }
  const int any_bad = __syncthreads_or(bad);  // also the barrier after the composites
  // kSmallSortGroup rows per workgroup (so that a few thousand rows spread over the whole device); a row's count
  // is split over 64 parts: the four sixteenths of a wave's lanes times the sixteen waves
  const int row_in_group = lane & (kSmallSortGroup - 1);
  const int split = part * (64 / kSmallSortGroup) + lane / kSmallSortGroup;
  constexpr int kParts = 16 * (64 / kSmallSortGroup);
  for (int r0 = blockIdx.x * kSmallSortGroup; r0 < npad; r0 += gridDim.x * kSmallSortGroup) {
    const int i = r0 + row_in_group;  // below npad: npad is a multiple of 128
    const double mine = comp[i];
    const double floor = mine - (double)(i & 0xFFF);  // the smallest composite of this key (unused for padding rows)
    // this part's share of the composites, in pairs (16-byte LDS reads)
    const int per = (((n + kParts - 1) / kParts) + 1) & ~1;
    const int e0 = split * per;
    const int e1 = min(e0 + per, (n + 1) & ~1);  // an odd n reads one composite of the padding: +inf
    int before = 0, smaller = 0;
#pragma unroll 8
    for (int e = e0; e < e1; e += 2) {
      const double2 c = *reinterpret_cast<const double2*>(comp + e);
      before += (c.x < mine) + (c.y < mine);
      smaller += (c.x < floor) + (c.y < floor);
    }
    share[0][split][row_in_group] = before;
    share[1][split][row_in_group] = smaller;
    __syncthreads();
    if (part == 0) {
      // lane = (row, quarter of the parts); the quarters are added across the lanes
      before = 0;
      smaller = 0;
      const int q0 = (lane / kSmallSortGroup) * (kParts / (64 / kSmallSortGroup));
#pragma unroll
      for (int p = 0; p < kParts / (64 / kSmallSortGroup); ++p) {
        before += share[0][q0 + p][row_in_group];
        smaller += share[1][q0 + p][row_in_group];
      }
#pragma unroll
      for (int off = kSmallSortGroup; off < 64; off <<= 1) {
        before += __shfl_xor(before, off);
        smaller += __shfl_xor(smaller, off);
      }
      if (lane < kSmallSortGroup) {
        if (i < n) {
          orig_of[before] = i;
          key_sorted[before] = (uint64_t)mine >> 12;
          kid_sorted[before] = (uint32_t)smaller;
          for (int k = 0; k < m; ++k) {
            const float v = value(i, k);
            xs[(int64_t)k * npad + i] = v;
            // -0.0 is stored as +0.0: every comparison reads the same, and differences of equal values are +0.0
            xs_sorted[(int64_t)k * npad + before] = v + 0.0f;
          }
        } else {
          orig_of[i] = -1;
          key_sorted[i] = ~0ull;
          kid_sorted[i] = (uint32_t)i;
          for (int k = 0; k < m; ++k) {
            xs[(int64_t)k * npad + i] = __uint_as_float(0x7FC00000u);
            xs_sorted[(int64_t)k * npad + i] = __uint_as_float(0x7FC00000u);
          }
        }
      }
    }
    __syncthreads();  // the shares are rewritten by the next row group
  }
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    SortParam sp;
    sp.kmin = 0ull;
    sp.shift = 0;
    sp.buckets = 0;
    sp.nonfinite = any_bad != 0;
    sp.totals_valid = 0;
    sp.orders_valid = 0;
    *param_out = sp;
  }
  const int64_t tid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  for (int64_t w = tid; w < n_zero_words; w += (int64_t)gridDim.x * blockDim.x) zero_words[w] = 0u;
}

enum DomVariant { kDomAuto = 0, kDomTwoCompares = 1, kDomKey64 = 2, kDomKey32 = 3, kDomArith = 4, kDomOrdersOnly = 5 };

// acc = (acc << 1) | bit, with the bit taken from a 64-lane mask: one v_addc_co_u32.
__device__ inline uint32_t shift_in(uint32_t acc, uint64_t mask) {
  uint32_t r;
  uint64_t carry_out;
  asm("v_addc_co_u32_e64 %0, %1, %2, %2, %3" : "=v"(r), "=s"(carry_out) : "v"(acc), "s"(mask));
  return r;
}

// acc = (acc << 1) | (o read as a signed integer is positive): v_med3_i32 clamps to 0..1, v_lshl_or_b32
// shifts it in.  Written out because the compiler turns the clamp into a compare and a select, and a
// compare that writes a lane mask issues at half the rate.
__device__ inline uint32_t shift_in_positive(uint32_t acc, uint32_t o) {
  uint32_t bit, r;
  asm("v_med3_i32 %0, %1, 0, 1" : "=v"(bit) : "v"(o));
  asm("v_lshl_or_b32 %0, %1, 1, %2" : "=v"(r) : "v"(acc), "v"(bit));
  return r;
}

// acc = (acc << 1) | (sign bit of o): one v_alignbit_b32 (the 64-bit value acc:o shifted right by 31).
__device__ inline uint32_t shift_in_sign(uint32_t acc, uint32_t o) {
  uint32_t r;
  asm("v_alignbit_b32 %0, %1, %2, 31" : "=v"(r) : "v"(acc), "v"(o));
  return r;
}

// 32 consecutive dominators ib .. ib+31 against the lane's row: bit t of the result says that
// dominator ib + t dominates the row.  The dominators' fitness and keys sit in SGPRs (M + 2 per
// dominator); from M = 4 on they are fetched G at a time with one scalar load per array, G shrinking
// as M grows, because once
// the SGPR file overflows the compiler spills through v_writelane / v_readlane, which is VALU work
// (measured: 3.5x the VALU instructions at M = 8 with 32 dominators in flight).
template <int M, int VARIANT>
__device__ inline uint32_t dominance_half_word(const float* __restrict__ xs, const uint64_t* __restrict__ key,
                                               const uint32_t* __restrict__ kid, int npad, int ib, const float (&xj)[M],
                                               uint64_t kj, uint32_t idj) {
  uint32_t acc = 0;
  if constexpr (M <= 3) {
    // few enough values per dominator for the compiler to schedule the scalar loads of all 32 itself
#pragma unroll
    for (int t = 31; t >= 0; --t) {
      const int i = ib + t;
      uint64_t c = ~0ull;
      if (VARIANT == kDomArith) {
        uint32_t o = 0u;
#pragma unroll
        for (int k = 0; k < M; ++k) o |= __float_as_uint(xj[k] - xs[(int64_t)k * npad + i]);
        acc = shift_in_sign(acc, o);  // some difference negative: this dominator is worse somewhere
        continue;
      }
      if (VARIANT == kDomKey32) {
        // all compares first, then a tree of ANDs: independent instructions for the scheduler
        uint64_t mk[M + 1];
#pragma unroll
        for (int k = 0; k < M; ++k) mk[k] = __builtin_amdgcn_ballot_w64(xs[(int64_t)k * npad + i] <= xj[k]);
        mk[M] = __builtin_amdgcn_ballot_w64(kid[i] != idj);
#pragma unroll
        for (int span = 1; span <= M; span *= 2)
#pragma unroll
          for (int k = 0; k + span <= M; k += 2 * span) mk[k] &= mk[k + span];
        acc = shift_in(acc, mk[0]);
        continue;
      }
#pragma unroll
      for (int k = 0; k < M; ++k) c &= __builtin_amdgcn_ballot_w64(xs[(int64_t)k * npad + i] <= xj[k]);
      if (VARIANT == kDomKey64) {
        c &= __builtin_amdgcn_ballot_w64(key[i] != kj);
      } else if (VARIANT == kDomKey32) {
        c &= __builtin_amdgcn_ballot_w64(kid[i] != idj);
      } else {
        uint64_t lt = 0ull;
#pragma unroll
        for (int k = 0; k < M; ++k) lt |= __builtin_amdgcn_ballot_w64(xs[(int64_t)k * npad + i] < xj[k]);
        c &= lt;
      }
      acc = shift_in(acc, c);
    }
  } else {
    constexpr int G = M <= 5 ? 8 : (M <= 8 ? 4 : 2);
#pragma unroll 1
    for (int g = 32 / G - 1; g >= 0; --g) {
      const int i0 = ib + g * G;  // wave-uniform
      float xi[M][G];
      uint64_t ki[G];
      uint32_t idi[G];
#pragma unroll
      for (int k = 0; k < M; ++k)
#pragma unroll
        for (int u = 0; u < G; ++u) xi[k][u] = xs[(int64_t)k * npad + i0 + u];
      if (VARIANT == kDomKey64) {
#pragma unroll
        for (int u = 0; u < G; ++u) ki[u] = key[i0 + u];
      }
      if (VARIANT == kDomKey32) {
#pragma unroll
        for (int u = 0; u < G; ++u) idi[u] = kid[i0 + u];
      }
#pragma unroll
      for (int u = G - 1; u >= 0; --u) {
        if (VARIANT == kDomArith) {
          uint32_t o = 0u;
#pragma unroll
          for (int k = 0; k < M; ++k) o |= __float_as_uint(xj[k] - xi[k][u]);
          acc = shift_in_positive(acc, o);
          continue;
        }
        uint64_t c = ~0ull;
#pragma unroll
        for (int k = 0; k < M; ++k) c &= __builtin_amdgcn_ballot_w64(xi[k][u] <= xj[k]);
        if (VARIANT == kDomKey64) {
          c &= __builtin_amdgcn_ballot_w64(ki[u] != kj);
        } else if (VARIANT == kDomKey32) {
          c &= __builtin_amdgcn_ballot_w64(idi[u] != idj);
        } else {
          uint64_t lt = 0ull;
#pragma unroll
          for (int k = 0; k < M; ++k) lt |= __builtin_amdgcn_ballot_w64(xi[k][u] < xj[k]);
          c &= lt;
        }
        acc = shift_in(acc, c);
      }
    }
  }
  if constexpr (VARIANT == kDomArith && M <= 3) {
    // (Up to three objectives; with more, the sign form measured no faster than clamp and shift-in: 200 000 x 8
    // 5.19 against 5.28 ms.  Three objectives: 65536 rows 260 -> 238 us, 20 000 rows 36.0 -> 34.2 us.)
    // The bits gathered say "worse than the row somewhere"; the others are no worse anywhere, and of those only
    // the rows equal to this one do not dominate it.  Equal rows have the row's key sum, so they -- and only rows
    // that are worse somewhere -- sit in the slots from kid(j) on: those bits go.  Only near the diagonal: kid
    // ascends with the slot, so the first lane holds the wave's smallest.
    acc = ~acc;
    if (ib + 32 > (int)__builtin_amdgcn_readfirstlane(idj)) {
      const int keep = (int)idj - ib;
      acc = keep <= 0 ? 0u : (keep >= 32 ? acc : acc & ((1u << keep) - 1u));
    }
  }
  return acc;
}


// The tile of block (bx, by): bx = one of ceil(npad / 256) groups of four 64-row waves, by = one of
// ceil(nwords / IW) column tiles.
// With tiles of two words the four waves of a block are two groups of rows times two neighbouring tiles: the two
// 16-byte pieces of a row then reach the cache from the same block at about the same time and leave it as one
// 32-byte sector (a block of four row groups and one tile wrote 50 MB for the 25 MB triangle of 20 000 x 3).
template <int M, int IW, int VARIANT>
__device__ __forceinline__ void dominance_tile(int bx, int by, const float* __restrict__ xs, const uint64_t* __restrict__ key,
                                      const uint32_t* __restrict__ kid, uint64_t* __restrict__ dom, int n, int npad,
                                      int64_t wstride, int nwords, const SortParam* __restrict__ param) {
  const int lane = threadIdx.x & 63;
  // (read from the first lane: the tile's first word depends on it, and the dominators are fetched by scalar loads
  // only at addresses that the compiler knows to be the same in every lane)
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int j = IW == 2 ? (bx * 2 + (wave >> 1)) * 64 + lane : (bx * 4 + wave) * 64 + lane;
  if (j - lane >= npad) return;  // whole wave past the padded population
  const int w0 = IW == 2 ? (by * 2 + (wave & 1)) * IW : by * IW;
  float xj[M];
#pragma unroll
  for (int k = 0; k < M; ++k) xj[k] = xs[(int64_t)k * npad + j];
  const uint64_t kj = key[j];
  const uint32_t idj = kid[j];
  const bool all_finite = VARIANT == kDomAuto && param->nonfinite == 0;  // wave-uniform
  uint64_t* __restrict__ out = dom + (int64_t)j * wstride;
  const int wend = (w0 + IW < nwords) ? w0 + IW : nwords;  // nwords = npad / 64 is even, and so is IW
  const int jlast = j - lane + 63;  // last row of this wave
  // Word pairs wholly above the diagonal (no row of a larger slot dominates these rows) are neither
  // evaluated nor stored: every reader bounds its scan of row j by the words up to j's own.
  // The results of the tile are kept in registers and stored together at the end, so that the 16-byte
  // pieces of one row reach the cache back to back and leave it as whole sectors.
  ulonglong2 res[IW / 2];
#pragma unroll
  for (int q = 0; q < IW / 2; ++q) res[q] = make_ulonglong2(0ull, 0ull);
#pragma unroll 1
  for (int p = 0; p < IW / 2; ++p) {
    const int w = w0 + 2 * p;
    if (w >= wend || w * 64 > jlast) break;
    uint32_t half[4];
    if (VARIANT == kDomAuto) {
      if (all_finite) {
#pragma unroll
        for (int h = 3; h >= 0; --h) half[h] = dominance_half_word<M, kDomArith>(xs, key, kid, npad, w * 64 + h * 32, xj, kj, idj);
        // padding dominators (i >= n) are NaN and give a NaN difference, whose sign is arbitrary: cleared here
        if (w * 64 + 128 > n) {
#pragma unroll
          for (int h = 0; h < 4; ++h) {
            const int first = w * 64 + h * 32;
            half[h] = first >= n ? 0u : (first + 32 > n ? half[h] & ((1u << (n - first)) - 1u) : half[h]);
          }
        }
      } else {
#pragma unroll
        for (int h = 3; h >= 0; --h) half[h] = dominance_half_word<M, kDomKey32>(xs, key, kid, npad, w * 64 + h * 32, xj, kj, idj);
      }
    } else {
#pragma unroll
      for (int h = 3; h >= 0; --h) {
        half[h] = dominance_half_word<M, VARIANT>(xs, key, kid, npad, w * 64 + h * 32, xj, kj, idj);
      }
    }
    // bits of padding rows (i >= n) are zero because their fitness is NaN
    const uint64_t lo = ((uint64_t)half[1] << 32) | half[0];
    const uint64_t hi = ((uint64_t)half[3] << 32) | half[2];
#pragma unroll
    for (int q = 0; q < IW / 2; ++q)
      if (q == p) res[q] = make_ulonglong2(lo, hi);
  }
  if (j < n) {
#pragma unroll
    for (int q = 0; q < IW / 2; ++q) {
      const int w = w0 + 2 * q;  // rows are 128-byte aligned and w is even: one 16-byte store per pair
      if (w < wend && w * 64 <= jlast) *reinterpret_cast<ulonglong2*>(out + w) = res[q];
    }
  }
}

// grid.x = ceil(npad / 256) blocks of four 64-row groups, grid.y = ceil(nwords / IW) column tiles (tiles of two words:
// ceil(npad / 128) blocks of two groups, ceil(nwords / 4) pairs of tiles).
template <int M, int IW, int VARIANT>
__global__ __launch_bounds__(256) void dominance_kernel(const float* __restrict__ xs, const uint64_t* __restrict__ key,
                                                        const uint32_t* __restrict__ kid, uint64_t* __restrict__ dom, int n,
                                                        int npad, int64_t wstride, int nwords,
                                                        const SortParam* __restrict__ param, int64_t ws_step) {
  to_population(ws_step, xs, key, kid, dom, param);
  dominance_tile<M, IW, VARIANT>((int)blockIdx.x, (int)blockIdx.y, xs, key, kid, dom, n, npad, wstride, nwords, param);
}

// The grid without the blocks above the diagonal, which are half of the rectangle above and return at once.  Tiles of
// two words: row block x (128 rows) needs x / 2 + 1 blocks of tiles, row block row_blocks - 1 - x the rest of about
// row_blocks / 2 + 2, so the two share column x of a grid of ceil(row_blocks / 2) x ((row_blocks - 1) / 2 + 2) blocks.
// Tiles of four words: row block x (256 rows) needs x + 1 tiles, the two together row_blocks + 1.
template <int M, int IW, bool MANY>
__global__ __launch_bounds__(256) void dominance_folded_kernel(const float* __restrict__ xs, const uint64_t* __restrict__ key,
                                                               const uint32_t* __restrict__ kid, uint64_t* __restrict__ dom,
                                                               int n, int npad, int64_t wstride, int nwords,
                                                               const SortParam* __restrict__ param, int row_blocks,
                                                               int64_t ws_step) {
  static_assert(IW == 2 || IW == 4, "tiles of two or four words");
  if constexpr (MANY) to_population(ws_step, xs, key, kid, dom, param);
  const int x = (int)blockIdx.x, y = (int)blockIdx.y;
  const int own = IW == 2 ? x / 2 + 1 : x + 1;
  int bx = x, by = y;
  if (y >= own) {
    bx = row_blocks - 1 - x;
    by = y - own;
    if (bx <= x || by > (IW == 2 ? bx / 2 : bx)) return;  // the middle row block has no partner; past the partner's diagonal
  }
  dominance_tile<M, IW, kDomAuto>(bx, by, xs, key, kid, dom, n, npad, wstride, nwords, param);
}

// The same matrix for a population that holds a NaN or an infinity, launched beside the kernels of prefix.hpp,
// which only handle finite populations: any grid, every block takes tiles in turn; nothing to do (and nothing
// done) when the population is finite.
template <int M>
__global__ __launch_bounds__(256) void dominance_nonfinite_kernel(const float* __restrict__ xs, const uint64_t* __restrict__ key,
                                                                  const uint32_t* __restrict__ kid, uint64_t* __restrict__ dom,
                                                                  int n, int npad, int64_t wstride, int nwords,
                                                                  const SortParam* __restrict__ param) {
  if (param->nonfinite == 0) return;
  const int gx = (npad + 255) / 256, gy = (nwords + 3) / 4;
  for (int64_t t = blockIdx.x; t < (int64_t)gx * gy; t += gridDim.x)
    dominance_tile<M, 4, kDomKey32>((int)(t % gx), (int)(t / gx), xs, key, kid, dom, n, npad, wstride, nwords, param);
}

// Any number of objectives (used above 8): same scheme, with the lane's own fitness re-read from
// memory for every objective instead of living in registers.
template <int IW>
__global__ __launch_bounds__(256) void dominance_any_m_kernel(const float* __restrict__ xs, const uint32_t* __restrict__ kid,
                                                              uint64_t* __restrict__ dom, int n, int npad, int64_t wstride,
                                                              int nwords, int m, int64_t ws_step) {
  to_population(ws_step, xs, kid, dom);
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int j = (blockIdx.x * 4 + wave) * 64 + lane;
  if (j - lane >= npad) return;
  const int w0 = blockIdx.y * IW;
  const uint32_t idj = kid[j];
  uint64_t* __restrict__ out = dom + (int64_t)j * wstride;
  const int wend = (w0 + IW < nwords) ? w0 + IW : nwords;
  const int jlast = j - lane + 63;
#pragma unroll 1
  for (int w = w0; w < wend; w += 2) {
    if (w * 64 > jlast) break;  // above the diagonal: never read
    uint32_t half[4];
#pragma unroll
    for (int h = 3; h >= 0; --h) {
      const int ib = w * 64 + h * 32;
      uint32_t acc = 0;
#pragma unroll 4
      for (int t = 31; t >= 0; --t) {
        const int i = ib + t;
        uint64_t c = __builtin_amdgcn_ballot_w64(kid[i] != idj);
        for (int k = 0; k < m; ++k) c &= __builtin_amdgcn_ballot_w64(xs[(int64_t)k * npad + i] <= xs[(int64_t)k * npad + j]);
        acc = shift_in(acc, c);
      }
      half[h] = acc;
    }
    if (j < n) {
      const uint64_t lo = ((uint64_t)half[1] << 32) | half[0];
      const uint64_t hi = ((uint64_t)half[3] << 32) | half[2];
      *reinterpret_cast<ulonglong2*>(out + w) = make_ulonglong2(lo, hi);
    }
  }
}

// ------------------------------------------------------------------ first front only

// mask[orig_of[j]] = 1 when no row dominates slot j, 0 otherwise: `non_dominate_rank(f) == 0`, the
// only thing src/evox/workflows/eval_monitor.py:301-302 and :333-335 keep of the ranks.  No matrix is
// built: a lane holds one row, the candidate dominators (slots below the end of the wave's own 64
// rows, since a dominator has a smaller key) stream past it 32 at a time in slot order, and the wave
// stops as soon as every one of its rows has met a dominator.  Rows of small key lie near the front and
// dominate most of the population, so almost every wave ends after its first few steps; a wave that
// holds a non-dominated row scans all the slots below it.
template <int M>
__global__ __launch_bounds__(256) void first_front_kernel(const float* __restrict__ xs, const uint64_t* __restrict__ key,
                                                          const uint32_t* __restrict__ kid, const int* __restrict__ orig_of,
                                                          int n, int npad, uint8_t* __restrict__ mask,
                                                          const Ctrl* __restrict__ ctrl, const SortParam* __restrict__ param,
                                                          int64_t ws_step) {
  // (several populations in the launch, one per blockIdx.z: their masks lie n bytes apart)
  to_population(ws_step, xs, key, kid, orig_of, ctrl, param);
  mask += (int64_t)blockIdx.z * n;
  const int lane = threadIdx.x & 63;
  const int j = (blockIdx.x * 4 + (threadIdx.x >> 6)) * 64 + lane;
  if (ctrl->err != 0) {  // the slot sort failed, nothing is valid: no row is reported (the status carries the error)
    if (j < n) mask[j] = 0;
    return;
  }
  if (j - lane >= n) return;  // npad is a multiple of 128: every row touched below exists
  float xj[M];
#pragma unroll
  for (int k = 0; k < M; ++k) xj[k] = xs[(int64_t)k * npad + j];
  const uint32_t idj = kid[j];
  const bool all_finite = param->nonfinite == 0;  // wave-uniform: the arithmetic form of the test applies
  bool dominated = j >= n;  // padding rows never hold the wave back
  const int iend = j - lane + 64;
#pragma unroll 1
  for (int ib = 0; ib < iend; ib += 32) {
    uint32_t h;
    if (all_finite) {
      h = dominance_half_word<M, kDomArith>(xs, key, kid, npad, ib, xj, 0ull, idj);
      // padding dominators (NaN) give differences of arbitrary sign
      if (ib + 32 > n) h = ib >= n ? 0u : h & ((1u << (n - ib)) - 1u);
    } else {
      h = dominance_half_word<M, kDomKey32>(xs, key, kid, npad, ib, xj, 0ull, idj);
    }
    dominated |= h != 0u;
    if (__builtin_amdgcn_ballot_w64(!dominated) == 0ull) break;
  }
  if (j < n) mask[orig_of[j]] = dominated ? 0 : 1;
}

// Any number of objectives (used above 8).
__global__ __launch_bounds__(256) void first_front_any_m_kernel(const float* __restrict__ xs, const uint32_t* __restrict__ kid,
                                                                const int* __restrict__ orig_of, int n, int npad, int m,
                                                                uint8_t* __restrict__ mask, const Ctrl* __restrict__ ctrl,
                                                                int64_t ws_step) {
  to_population(ws_step, xs, kid, orig_of, ctrl);
  mask += (int64_t)blockIdx.z * n;
  const int lane = threadIdx.x & 63;
  const int j = (blockIdx.x * 4 + (threadIdx.x >> 6)) * 64 + lane;
  if (ctrl->err != 0) {
    if (j < n) mask[j] = 0;
    return;
  }
  if (j - lane >= n) return;
  const uint32_t idj = kid[j];
  bool dominated = j >= n;
  const int iend = j - lane + 64;
#pragma unroll 1
  for (int ib = 0; ib < iend; ib += 32) {
    uint64_t any = 0ull;
#pragma unroll 4
    for (int t = 0; t < 32; ++t) {
      const int i = ib + t;
      uint64_t c = __builtin_amdgcn_ballot_w64(kid[i] != idj);
      for (int k = 0; k < m; ++k) c &= __builtin_amdgcn_ballot_w64(xs[(int64_t)k * npad + i] <= xs[(int64_t)k * npad + j]);
      any |= c;
    }
    dominated |= ((any >> lane) & 1ull) != 0ull;
    if (__builtin_amdgcn_ballot_w64(!dominated) == 0ull) break;
  }
  if (j < n) mask[orig_of[j]] = dominated ? 0 : 1;
}

}  // namespace evx
