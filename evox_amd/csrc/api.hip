// C ABI of libevox_hip.so (declared in include/evox_hip.h): argument checks, workspace layout
// and kernel launches.  Nothing here allocates device memory or waits for the device, except
// evox_hip_read_status(); the selection entry points keep 64 bytes of pinned host memory per device (outcome_slot).
#include <string.h>

#include <atomic>
#include <mutex>
#include <new>
#include <type_traits>

#include "../../include/evox_hip.h"
#include "batched.hpp"
#include "calibrate.hpp"
#include "common.hpp"
#include "crowd.hpp"
#include "dominance.hpp"
#include "finish.hpp"
#include "hv.hpp"
#include "order.hpp"
#include "peel.hpp"
#include "peel_lds.hpp"
#include "prefix.hpp"
#include "radix.hpp"
#include "stepped.hpp"
#include "two.hpp"
#include "two_small.hpp"
#include "wide.hpp"

namespace evx {

constexpr int kMaxGrid = 4096;  // slots of the grid barrier
constexpr int kRecordsMaxRows = 65534;       // largest population whose record units hold three 16-bit slots
constexpr int kRecordsMaxRowsWide = 262144;  // largest population peeled with the record protocol at all (two
                                             // 24-bit slots per unit; 128 blocks of 8 waves own 256 rows per wave)

struct Options {
  int peel_blocks_per_cu = 2;
  int peel_witness = 1;
  int peel_record_blocks = 0;  // sweeping blocks of the record protocol, 16 .. 255 (plus the lister); 0 = by size
  int peel_records = 1;  // record protocol (all-to-all, no master) for populations up to kRecordsMaxRowsWide
  int peel_lds = 1;      // populations whose lower triangle fits the LDS of the device are peeled from LDS (peel_lds.hpp)
  int peel_lds_blocks = 0;  // sweeping workgroups of that kernel, 0 = by size
  int peel_stepped = 0;     // 1: the fronts are peeled one launch each by kernels that never wait for each other (stepped.hpp),
                            // and the last front is ordered likewise; 0: only where the persistent grids cannot be resident
  int64_t two_small_min_rows = 128;  // populations of two objectives and at least this many rows (at most 4096) that go to a
                                   // one-workgroup kernel take the one without a matrix (two_small.hpp); 0 = never
  int64_t two_min_rows = 4097;  // populations of two objectives and at least this many rows are ranked without a matrix (two.hpp); 0 = never
  int64_t two_min_rows_partial = 4097;  // ... when the ranking may stop at the front that holds a given row (measured, us per
                                        // selection of half the rows, without / with a matrix: 5000 rows 110 / 178, 20 000 rows
                                        // 218 / 362, 50 000 rows 324 / 1181; all ranks: 5000 rows 140 / 332)
  int peel_tail = 1;        // that kernel also orders a small last front (0: always the kernels of finish.hpp)
  int tail_merged = 1;      // after such a peel, ordering (where still needed) and gather share one launch
  int launch_memory = 1;    // ... unless the last selection of this shape had a last front that the peel left alone
  unsigned spin_limit = 4000000u;
  int dominance_tile_words = 0;  // 0 = by size (2 or 4)
  int dominance_folded = 1;      // tiles of two words: only the blocks at or below the diagonal are launched
  int mid_argsort = 1;  // an argsort step of 8193 .. kMidArgsortRows positions in one kernel without waits (0: the radix sort)
  int small_sort = 1;  // populations up to kSmallSortRows rows are put in slot order by one kernel (0: bucket sort)
  int64_t prefix_min_rows = 65536;  // finite populations of at least this many rows and 3 objectives (a quarter more
                                    // with 2, fewer with more: 28672 at 8, 10240 at 16 -- prefix_least_rows) get
                                    // their matrix from the per-objective orders (prefix.hpp); 0 = never
  int64_t prefix_double_tile = 131072;  // order-based matrix, up to four objectives: from this many rows on a workgroup
                                        // takes both tiles of a 128-byte line; 0 = never
  int prefix_mode = 3;  // measurements: 1 = popcounts only, 2 = matrix only
  int prefix_bands = 1;  // stretches of the order-based matrix: 1 = bands of rows counted from row 0, 0 = from each tile's diagonal
  int batched_stage = 1;  // the one-workgroup kernel reads its dominators from a copy of the fitness in LDS when the populations
                          // have at most 256 rows and are no more than the device has compute units (0: by scalar loads always)
  int order_stream = 1;  // the per-objective orders of more than 32768 rows come from workgroups that sort shares of
                         // them in LDS (0: from the radix sort whose workgroups wait for each other)
  int order_stream_capacity = 16384;  // entries that such a workgroup sorts at once (tests make it small: shares in pieces)
  int prefix_count_first = 1;  // a selection whose last two of this shape found all they keep in front 0 has the order-based
                               // kernel count dominators first and build the matrix only if front 0 falls short; 0 = never
};
static Options g_opt;
// The tunables that calls made from this thread use: those handed to evox_hip_options_use, else the process-wide ones.
static thread_local const Options* t_opt = nullptr;
static inline const Options& opt() { return t_opt != nullptr ? *t_opt : g_opt; }


struct Layout {
  int n, m, npad, nwords, kstride, buckets, prep_blocks;
  int64_t wstride;
  // byte offsets
  size_t ctrl, fsize, fronts_slot, fronts_orig, hist, zero_end, fstart, xs, key, partials, sortparam, bstart, bcursor,
      scanflags, tailbuf, records, two_ring, members, member_key, slot_of, xs_sorted, key_sorted, kid_sorted, orig_of, count, witness, total0, witness0, rank, dist, perm, order, rpairs0, rpairs1, rtable, rtotals, pos, scost, dkey, wide, wide_bytes, dom, total;
};

static size_t align_up(size_t v) { return (v + 255) / 256 * 256; }
static size_t wide_workspace_need(int64_t n, int64_t m);  // (workspace of the kernels of wide.hpp, defined with them)
constexpr int kErrNotResident = -100;  // internal: the grid of a persistent kernel would not be resident at once

static bool make_layout(int64_t n, int64_t m, Layout* L) {
  if (n < 1 || m < 1 || n > 0x7FFFFF00ll || m > 65535) return false;
  L->n = (int)n;
  L->m = (int)m;
  L->npad = (int)round_up(n, 128);
  // the objectives are columns npad floats apart: at a multiple of 16 KB the same row of six or more columns
  // competes for one set of the scalar cache (pairwise matrix of 65536 rows x 8: 1.19 ms, of 49152 rows: 0.42 ms)
  if (L->npad % 4096 == 0 && n >= 16384) L->npad += 128;
  L->nwords = L->npad / 64;
  L->wstride = round_up(L->nwords, 16);
  L->kstride = (int)round_up(n, 64);
  // buckets of the slot sort: a power of two near 4 n, between 1024 and 65536
  int buckets = 1024;
  while (buckets < 65536 && buckets < 4 * n) buckets <<= 1;
  L->buckets = buckets;
  L->prep_blocks = (int)((L->npad + 255) / 256 < 1024 ? (L->npad + 255) / 256 : 1024);
  size_t o = 0;
  // --- cleared on every call: control block, front sizes, front bitmaps, sort histogram
  L->ctrl = o;        o = align_up(o + sizeof(Ctrl) + sizeof(unsigned long long) * kMaxGrid);
  L->fsize = o;       o = align_up(o + sizeof(int) * (size_t)(n + 2));
  L->fronts_slot = o; o = align_up(o + sizeof(uint64_t) * kFrontBuffers * kFrontStride * (size_t)L->nwords);
  L->fronts_orig = o; o = align_up(o + sizeof(uint64_t) * kFrontBuffers * kFrontStride * (size_t)L->nwords);
  L->hist = o;        o = align_up(o + sizeof(int) * (size_t)buckets);
  L->scanflags = o;   o = align_up(o + sizeof(unsigned long long) * 64);
  L->tailbuf = o;     o = align_up(o + (n <= 32768 ? sizeof(unsigned long long) * kTailCopies * kTailRows : 0));
  L->records = o;     o = align_up(o + (n <= 32768 ? sizeof(unsigned long long) * kLdsPeelRecordUnits : (n <= kRecordsMaxRowsWide ? sizeof(unsigned long long) * kRecRing * (n > kRecordsMaxRows ? kRecUnitsWide : kRecUnits) : 0)));
  // the hand-over rings of the two-objective ranking (two.hpp)
  L->two_ring = o;    o = align_up(o + (m == 2 && n <= kTwoMaxRows ? sizeof(unsigned long long) * kTwoRingStride * (size_t)((n + kTwoChunk - 1) / kTwoChunk) : 0));
  L->zero_end = o;
  L->fstart = o;     o = align_up(o + sizeof(int) * (size_t)(n + 2));
  L->xs = o;         o = align_up(o + sizeof(float) * (size_t)m * L->npad);
  L->key = o;        o = align_up(o + sizeof(uint64_t) * (size_t)L->npad);
  L->partials = o;   o = align_up(o + sizeof(unsigned long long) * 3 * (size_t)L->prep_blocks);
  L->sortparam = o;  o = align_up(o + sizeof(SortParam));
  L->bstart = o;     o = align_up(o + sizeof(int) * (size_t)(buckets + 1));
  L->bcursor = o;    o = align_up(o + sizeof(int) * (size_t)buckets);
  L->members = o;    o = align_up(o + sizeof(int) * (size_t)n);
  L->member_key = o; o = align_up(o + sizeof(uint64_t) * (size_t)n);
  L->xs_sorted = o;  o = align_up(o + sizeof(float) * (size_t)m * L->npad);
  L->key_sorted = o; o = align_up(o + sizeof(uint64_t) * (size_t)L->npad);
  L->kid_sorted = o; o = align_up(o + sizeof(uint32_t) * (size_t)L->npad);
  L->orig_of = o;    o = align_up(o + sizeof(int) * (size_t)L->npad);
  L->slot_of = o;    o = align_up(o + sizeof(int) * (size_t)n);
  L->count = o;      o = align_up(o + sizeof(int) * (size_t)n);
  L->witness = o;    o = align_up(o + sizeof(int) * (size_t)n);
  // popcount and highest non-empty word of every row as the order-based dominance kernel leaves them (kept apart
  // from count / witness, which the peel consumes, so that the count stage can be repeated)
  L->total0 = o;     o = align_up(o + sizeof(int) * (size_t)n);
  L->witness0 = o;   o = align_up(o + sizeof(int) * (size_t)n);
  L->rank = o;       o = align_up(o + sizeof(int) * (size_t)n);
  L->dist = o;       o = align_up(o + sizeof(float) * (size_t)n);
  L->perm = o;       o = align_up(o + sizeof(int) * (size_t)n);
  L->order = o;      o = align_up(o + sizeof(int) * (size_t)n);
  // radix sort of large fronts: only populations that can have one get the buffers
  const size_t rseg = n > kRadixMinCandidates ? (size_t)m * L->kstride : 0;
  L->rpairs0 = o;    o = align_up(o + sizeof(unsigned long long) * rseg);
  L->rpairs1 = o;    o = align_up(o + sizeof(unsigned long long) * rseg);
  L->rtable = o;     o = align_up(o + (rseg ? sizeof(int) * (size_t)m * 256 * kRadixMaxWorkers : 0));
  L->rtotals = o;    o = align_up(o + (rseg ? sizeof(int) * (size_t)m * 256 : 0));
  L->pos = o;        o = align_up(o + sizeof(int) * (size_t)m * L->kstride);
  L->scost = o;      o = align_up(o + sizeof(float) * (size_t)m * L->kstride);
  L->dkey = o;       o = align_up(o + sizeof(uint32_t) * (size_t)L->kstride);
  L->dom = o;        o = align_up(o + sizeof(uint64_t) * (size_t)n * (size_t)L->wstride);
  // behind the matrix (the entry points that build none need only the bytes before it): the ordering of the last
  // front by kernels that never wait for each other (the tail of the stepped path)
  L->wide_bytes = wide_workspace_need(n, m);
  L->wide = o;       o = align_up(o + L->wide_bytes);
  L->total = o;
  return true;
}

struct Ws {
  Layout L;
  uint8_t* base;
  // several populations of one shape in the same launches (blockIdx.z): `step` bytes from the workspace of one to that
  // of the next, all laid out alike; 1 and 0 for a single population
  int batch = 1;
  int64_t step = 0;
  // above zero: the order-based dominance kernel has only counted so far; the count stage launches it again for the
  // matrix, and that launch does nothing when front 0 holds this many rows
  mutable int64_t matrix_unless = 0;
  template <class T>
  T* at(size_t off) const {
    return reinterpret_cast<T*>(base + off);
  }
  Ctrl* ctrl() const { return at<Ctrl>(L.ctrl); }
};

// The bit matrix and what lies behind it are the last regions: entry points that never build it need only the bytes before it.
static int open_ws(int64_t n, int64_t m, void* ws, size_t bytes, Ws* out, bool with_matrix = true) {
  if (!make_layout(n, m, &out->L)) return kErrBadArg;
  const size_t need = with_matrix ? out->L.total : out->L.dom;
  if (ws == nullptr || bytes < need || (reinterpret_cast<uintptr_t>(ws) & 255u) != 0) return kErrWorkspace;
  out->base = static_cast<uint8_t*>(ws);
  return 0;
}

// (The small host-side caches below are read and written by whichever threads call into the library: each slot is
// an atomic that holds a value derived from the device alone, so two threads that fill it at once store the same.)
static int device_cus() {
  static std::atomic<int> cached[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  int v = cached[dev].load(std::memory_order_relaxed);
  if (v == 0) {
    if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0) v = 256;
    cached[dev].store(v, std::memory_order_relaxed);
  }
  return v;
}

// What the last selections on this device found, for the choice of launches of the next one: sixteen words of pinned
// host memory per device, which the last kernel of a selection writes (1: the peel kernel ordered the last front, 2: it
// left it to the ordering kernels) and the host reads at its next call of that shape without waiting for anything --
// a stale or missing word costs a few microseconds, never a result.  Allocated at the first selection on a device
// that may allocate (not during a stream capture); null until then and for callers that may not.
// salt: 0 for the selections of 4-byte fitness, 1 for those whose last front is ordered by the kernels of wide.hpp
// (there the word says whether that front was small, 1, or large, 2), 2 for whether front 0 alone held what was kept
// (GatherArgs::front0_note).
static int* outcome_slot(int64_t n, int64_t m, bool may_allocate, hipStream_t s, int salt = 0) {
  static std::atomic<int*> words[64];
  static std::atomic<bool> failed[64];
  static std::mutex mu;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return nullptr;
  int* base = words[dev].load(std::memory_order_acquire);
  if (base == nullptr) {
    if (!may_allocate || failed[dev].load(std::memory_order_relaxed)) return nullptr;
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(s, &capturing) != hipSuccess || capturing != hipStreamCaptureStatusNone) {
      (void)hipGetLastError();
      return nullptr;
    }
    std::lock_guard<std::mutex> lock(mu);
    base = words[dev].load(std::memory_order_acquire);
    if (base == nullptr) {
      void* p = nullptr;
      if (hipHostMalloc(&p, 64, hipHostMallocDefault) != hipSuccess || p == nullptr) {
        (void)hipGetLastError();
        failed[dev].store(true, std::memory_order_relaxed);
        return nullptr;
      }
      memset(p, 0, 64);
      base = static_cast<int*>(p);
      words[dev].store(base, std::memory_order_release);
    }
  }
  return base + (int)(((uint64_t)n * 31u + (uint64_t)m + (uint64_t)salt * 7u) & 15u);
}

#define EVX_LAUNCH_CHECK()                          \
  do {                                              \
    hipError_t e_ = hipGetLastError();              \
    if (e_ != hipSuccess) return (int)e_;           \
  } while (0)

// ------------------------------------------------------------------ stages

template <int M, int IW>
static void launch_dominance_m(const Ws& w, int variant, hipStream_t s) {
  const Layout& L = w.L;
  dim3 grid((L.npad + 255) / 256, (L.nwords + IW - 1) / IW, w.batch);
  if (IW == 2) grid = dim3((L.npad + 127) / 128, (L.nwords + 3) / 4, w.batch);  // a block = two row groups x two tiles
  auto launch = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, grid, dim3(256), 0, s, w.at<float>(L.xs_sorted), w.at<uint64_t>(L.key_sorted),
                       w.at<uint32_t>(L.kid_sorted), w.at<uint64_t>(L.dom), L.n, L.npad, L.wstride, L.nwords,
                       w.at<SortParam>(L.sortparam), w.step);
  };
  if ((IW == 2 || IW == 4) && variant == kDomAuto && opt().dominance_folded) {
    const int row_blocks = IW == 2 ? (L.npad + 127) / 128 : (L.npad + 255) / 256;
    const int column = IW == 2 ? (row_blocks - 1) / 2 + 2 : row_blocks + 1;
    auto folded = [&](auto kernel) {
      hipLaunchKernelGGL(kernel, dim3((row_blocks + 1) / 2, column, w.batch), dim3(256), 0, s, w.at<float>(L.xs_sorted),
                         w.at<uint64_t>(L.key_sorted), w.at<uint32_t>(L.kid_sorted), w.at<uint64_t>(L.dom), L.n, L.npad, L.wstride,
                         L.nwords, w.at<SortParam>(L.sortparam), row_blocks, w.step);
    };
    if (w.batch > 1)
      folded(dominance_folded_kernel<M, (IW == 2 ? 2 : 4), true>);
    else
      folded(dominance_folded_kernel<M, (IW == 2 ? 2 : 4), false>);
    return;
  }
  switch (variant) {
    case kDomTwoCompares: launch(dominance_kernel<M, IW, kDomTwoCompares>); break;
    case kDomKey64: launch(dominance_kernel<M, IW, kDomKey64>); break;
    case kDomKey32: launch(dominance_kernel<M, IW, kDomKey32>); break;
    default: launch(dominance_kernel<M, IW, kDomAuto>); break;
  }
}

template <int IW>
static void launch_dominance(const Ws& w, int variant, hipStream_t s) {
  const Layout& L = w.L;
  switch (L.m) {
    case 1: launch_dominance_m<1, IW>(w, variant, s); break;
    case 2: launch_dominance_m<2, IW>(w, variant, s); break;
    case 3: launch_dominance_m<3, IW>(w, variant, s); break;
    case 4: launch_dominance_m<4, IW>(w, variant, s); break;
    case 5: launch_dominance_m<5, IW>(w, variant, s); break;
    case 6: launch_dominance_m<6, IW>(w, variant, s); break;
    case 7: launch_dominance_m<7, IW>(w, variant, s); break;
    case 8: launch_dominance_m<8, IW>(w, variant, s); break;
    default: {
      // nine to sixteen objectives: the register kernel in its production form (tiles of four words, form chosen
      // on the device); the other tile sizes and the check variants, and more objectives, take the generic kernel
      if (IW == 4 && variant == kDomAuto && L.m <= 16) {
        auto wide = [&](auto kernel) {
          hipLaunchKernelGGL(kernel, dim3((L.npad + 255) / 256, (L.nwords + 3) / 4, w.batch), dim3(256), 0, s, w.at<float>(L.xs_sorted),
                             w.at<uint64_t>(L.key_sorted), w.at<uint32_t>(L.kid_sorted), w.at<uint64_t>(L.dom), L.n, L.npad,
                             L.wstride, L.nwords, w.at<SortParam>(L.sortparam), w.step);
        };
        switch (L.m) {
          case 9: wide(dominance_kernel<9, 4, kDomAuto>); return;
          case 10: wide(dominance_kernel<10, 4, kDomAuto>); return;
          case 11: wide(dominance_kernel<11, 4, kDomAuto>); return;
          case 12: wide(dominance_kernel<12, 4, kDomAuto>); return;
          case 13: wide(dominance_kernel<13, 4, kDomAuto>); return;
          case 14: wide(dominance_kernel<14, 4, kDomAuto>); return;
          case 15: wide(dominance_kernel<15, 4, kDomAuto>); return;
          default: wide(dominance_kernel<16, 4, kDomAuto>); return;
        }
      }
      dim3 grid((L.npad + 255) / 256, (L.nwords + IW - 1) / IW, w.batch);
      hipLaunchKernelGGL((dominance_any_m_kernel<IW>), grid, dim3(256), 0, s, w.at<float>(L.xs_sorted),
                         w.at<uint32_t>(L.kid_sorted), w.at<uint64_t>(L.dom), L.n, L.npad, L.wstride, L.nwords, L.m, w.step);
    }
  }
}

template <int M>
static void launch_first_front(const Ws& w, uint8_t* mask, hipStream_t s) {
  const Layout& L = w.L;
  hipLaunchKernelGGL((first_front_kernel<M>), dim3((L.n + 255) / 256, 1, w.batch), dim3(256), 0, s, w.at<float>(L.xs_sorted),
                     w.at<uint64_t>(L.key_sorted), w.at<uint32_t>(L.kid_sorted), w.at<int>(L.orig_of), L.n, L.npad, mask,
                     w.ctrl(), w.at<SortParam>(L.sortparam), w.step);
}

// Fitness -> structure of arrays + keys, state reset, then the slot sort (order.hpp).
// A population given in one part (n_first == n, second part unused) or in two.
struct Fitness {
  const float* f;
  int64_t sr, sc;
  int64_t n_first;
  const float* f2;
  int64_t sr2, sc2;
  int64_t step = 0, step2 = 0;  // several populations: elements from one population's fitness to the next one's
};

static Fitness one_part(const float* f, int64_t n, int64_t sr, int64_t sc, int64_t step = 0) {
  return Fitness{f, sr, sc, n, f, sr, sc, step, step};
}

static int stage_prepare(const Ws& w, const Fitness& src, bool with_sort, hipStream_t s, bool lexicographic = false) {
  const Layout& L = w.L;
  if (src.f == nullptr || src.f2 == nullptr || src.n_first < 0 || src.n_first > L.n) return kErrBadArg;
  const int64_t zero_words = (int64_t)((L.zero_end - L.ctrl) / 4);
  // (every workgroup of small_sort_kernel reads its whole population to place sixteen rows: with several populations
  // in the launch, more workgroups than the device holds at once take turns -- 16 x 4096 rows: 102 us against 10 for
  // one population, the five launches of the bucket sort 30)
  const bool many = w.batch > 1;
  const bool small_sort_pays = w.batch == 1 || (int64_t)w.batch * (L.npad / kSmallSortGroup) <= 2 * device_cus();
  if (with_sort && !lexicographic && L.n <= kSmallSortRows && L.m <= kSmallSortObjectives && (int64_t)L.n * L.m <= kSmallSortValues &&
      opt().small_sort && small_sort_pays) {
    auto launch = [&](auto kernel) {
      hipLaunchKernelGGL(kernel, dim3(L.npad / kSmallSortGroup, 1, w.batch), dim3(kSmallSortThreads), sizeof(double) * (size_t)L.npad, s, src.f,
                         src.sr, src.sc, (int)src.n_first, src.f2, src.sr2, src.sc2, L.n, L.m, L.npad, w.at<float>(L.xs),
                         w.at<SortParam>(L.sortparam), w.at<uint64_t>(L.key_sorted), w.at<uint32_t>(L.kid_sorted),
                         w.at<float>(L.xs_sorted), w.at<int>(L.orig_of), w.at<uint32_t>(L.ctrl), zero_words, src.step, src.step2, w.step);
    };
    if (many)
      launch(small_sort_kernel<true>);
    else
      launch(small_sort_kernel<false>);
    EVX_LAUNCH_CHECK();
    return 0;
  }
  auto launch_prepare = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, dim3(L.prep_blocks, 1, w.batch), dim3(256), 0, s, src.f, src.sr, src.sc, (int)src.n_first, src.f2,
                       src.sr2, src.sc2, L.n, L.m, L.npad, w.at<float>(L.xs), w.at<uint64_t>(L.key),
                       w.at<unsigned long long>(L.partials), w.at<uint32_t>(L.ctrl), zero_words, lexicographic ? 1 : 0, src.step,
                       src.step2, w.step);
  };
  if (many)
    launch_prepare(prepare_kernel<true>);
  else
    launch_prepare(prepare_kernel<false>);
  EVX_LAUNCH_CHECK();
  if (!with_sort) return 0;
  int blocks = (L.n + 255) / 256;
  if (blocks > 2048) blocks = 2048;
  auto launch_hist = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, dim3(blocks, 1, w.batch), dim3(256), 0, s, w.at<uint64_t>(L.key), L.n,
                       w.at<unsigned long long>(L.partials), L.prep_blocks, L.buckets, w.at<int>(L.hist),
                       w.at<SortParam>(L.sortparam), w.step);
  };
  if (many)
    launch_hist(bucket_hist_kernel<true>);
  else
    launch_hist(bucket_hist_kernel<false>);
  EVX_LAUNCH_CHECK();
  auto launch_scan = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, dim3(L.buckets / 1024, 1, w.batch), dim3(256), 0, s, w.at<int>(L.hist), L.buckets,
                       w.at<int>(L.bstart), w.at<int>(L.bcursor), w.at<unsigned long long>(L.scanflags), w.ctrl(), w.step);
  };
  if (many)
    launch_scan(bucket_scan_kernel<true>);
  else
    launch_scan(bucket_scan_kernel<false>);
  EVX_LAUNCH_CHECK();
  auto launch_scatter = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, dim3(blocks, 1, w.batch), dim3(256), 0, s, w.at<uint64_t>(L.key), L.n,
                       w.at<SortParam>(L.sortparam), w.at<int>(L.bcursor), w.at<int>(L.members), w.at<uint64_t>(L.member_key),
                       w.ctrl(), w.step);
  };
  if (many)
    launch_scatter(bucket_scatter_kernel<true>);
  else
    launch_scatter(bucket_scatter_kernel<false>);
  EVX_LAUNCH_CHECK();
  int pblocks = (L.npad + 255) / 256;
  if (pblocks > 2048) pblocks = 2048;
  auto launch_place = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, dim3(pblocks, 1, w.batch), dim3(256), 0, s, w.at<float>(L.xs), L.n, L.m,
                       L.npad, w.at<SortParam>(L.sortparam), w.at<int>(L.bstart), w.at<int>(L.members), w.at<uint64_t>(L.member_key),
                       w.at<uint64_t>(L.key_sorted), w.at<uint32_t>(L.kid_sorted), w.at<float>(L.xs_sorted), w.at<int>(L.orig_of), w.at<int>(L.slot_of),
                       w.ctrl(), w.step);
  };
  if (many)
    launch_place(bucket_place_kernel<true>);
  else
    launch_place(bucket_place_kernel<false>);
  EVX_LAUNCH_CHECK();
  return 0;
}

// From how many rows on the matrix comes from the per-objective orders: the pairwise kernel's work grows with the
// objectives (two compares each per pair), the other's hardly does, and it starts from some 160 us for the orders
// themselves.  Measured, a whole selection of uniform fitness in us, pairwise / from the orders:
//   x 3: 60 000 521 / 530;  x 4: 40 000 300 / 337, 50 000 406 / 376;  x 5: 40 000 295 / 335, 50 000 395 / 350;
//   x 6: 40 000 325 / 343, 50 000 439 / 352;  x 7: 33 000 302 / 315, 40 000 377 / 351;  x 8: 26 000 254 / 312,
//   33 000 335 / 325, 50 000 584 / 386;  x 9: 20 000 251 / 305, 26 000 342 / 323;  x 10: 20 000 269 / 315, 26 000 363 / 329;
//   x 12: 16 000 261 / 308, 20 000 312 / 307;  x 14: 16 000 301 / 327, 20 000 363 / 327;  x 16: 12 000 253 / 330,
//   16 000 342 / 344, 20 000 424 / 352;  x 2 (65 536 rows): 227 / 239, (100 000) 558 / 370.
// As thirty-seconds of the tunable (65 536 rows for three objectives):
// Up to kMidArgsortRows rows the orders come from workgroups that sort in LDS and cost 60 to 90 us less:
//   x 8: 26 000 254 / 261, 32 768 322 / 295;  x 9: 16 000 212 / 224, 20 000 252 / 236;  x 10: 16 000 222 / 231,
//   20 000 268 / 245;  x 12: 12 000 198 / 210, 16 000 257 / 225;  x 16: 9000 220 / 215, 12 000 259 / 237.
static int64_t prefix_least_rows(int m) {
  int parts = m <= 2 ? 40 : m == 3 ? 32 : m <= 5 ? 22 : m == 6 ? 20 : m == 7 ? 18 : m == 8 ? 16 : m <= 10 ? 12 : m <= 12 ? 10 : m <= 14 ? 9 : 8;
  if (opt().mid_argsort && m >= 8) parts = m == 8 ? 14 : m <= 10 ? 9 : m <= 12 ? 7 : m <= 14 ? 6 : 5;
  return opt().prefix_min_rows / 32 * parts + (opt().prefix_min_rows % 32 != 0 ? 1 : 0);
}
static bool prefix_dominance_applies(const Layout& L) {
  if (opt().prefix_min_rows <= 0 || L.m < 2 || L.m > kPrefixMaxObjectives) return false;
  return L.n >= prefix_least_rows(L.m) && L.n > kRadixMinCandidates && L.n <= kPrefixMaxRows;
}
static int stage_dominance_prefix(const Ws& w, bool orders_only, hipStream_t s, int64_t count_first = 0);
static int dispatch_dominance_prefix(const Ws& w, hipStream_t s, int phase = 0);

static int dominance_tile_words(const Layout& L) {
  const int tile = opt().dominance_tile_words;
  if (tile != 0) return tile;
  return L.m >= 2 && L.m <= 8 && L.n <= (L.m >= 6 ? 32768 : 24576) ? 2 : 4;
}

// count_first: above zero, the caller keeps that many rows and expects front 0 to hold them (see Ws::matrix_unless).
static int stage_dominance(const Ws& w, int variant, hipStream_t s, int64_t count_first = 0) {
  // (kDomOrdersOnly: the first half of the path below alone, for measurements of the second)
  if (variant == kDomOrdersOnly) return prefix_dominance_applies(w.L) ? stage_dominance_prefix(w, true, s) : kErrBadArg;
  // (the orders of that path come from kernels whose workgroups wait for each other: not with the stepped path)
  // (nor for several populations in one launch: those orders come from a grid that fills the device)
  if (variant == kDomAuto && prefix_dominance_applies(w.L) && !opt().peel_stepped && w.batch == 1) return stage_dominance_prefix(w, false, s, count_first);
  // (the lower triangle in tiles of 4 words keeps every SIMD busy with several waves; up to about 24 000 rows of
  // two to eight objectives tiles of 2 words leave a shorter half-empty tail -- measured, us, tiles of 2 / 4:
  // 5000 x 3: 5.8 / 7.9, 16 000 x 3: 20.3 / 25.7, 20 000 x 2: 20.6 / 23.1, x 3: 27.6 / 31.3, x 8: 64.3 / 80.8,
  // 24 000 x 3: 38.8 / 39.8, 28 000 x 3: 49.1 / 48.1, x 8: 110.8 / 132.1, 50 000 x 3: 147.5 / 138.4 --; 8 and 16
  // are kept for measurements)
  const int tile = dominance_tile_words(w.L);
  if (tile >= 16)
    launch_dominance<16>(w, variant, s);
  else if (tile >= 8)
    launch_dominance<8>(w, variant, s);
  else if (tile >= 4)
    launch_dominance<4>(w, variant, s);
  else
    launch_dominance<2>(w, variant, s);
  EVX_LAUNCH_CHECK();
  return 0;
}

static int stage_count(const Ws& w, bool fill_dist, hipStream_t s, bool need_counts) {
  const Layout& L = w.L;
  int blocks = (L.n + 3) / 4;
  const int cap = device_cus() * 8;
  if (blocks > cap) blocks = cap;
  hipLaunchKernelGGL(count_kernel, dim3(blocks), dim3(256), 0, s, w.at<uint64_t>(L.dom), L.wstride, L.n,
                     w.at<int>(L.orig_of), w.at<int>(L.count), w.at<int>(L.rank), w.at<int>(L.witness),
                     w.at<uint64_t>(L.fronts_slot), w.at<uint64_t>(L.fronts_orig), w.at<int>(L.fsize),
                     fill_dist ? w.at<float>(L.dist) : (float*)nullptr, w.ctrl(), w.at<SortParam>(L.sortparam), need_counts ? 1 : 0);
  EVX_LAUNCH_CHECK();
  if (prefix_dominance_applies(L)) {
    // the order-based dominance kernel has left the popcounts: count_kernel above returned at once (the choice is
    // made on the device: a population with a NaN or an infinity went through the pairwise kernel and is counted there)
    hipLaunchKernelGGL(count_from_totals_kernel, dim3((L.n + 255) / 256 < 128 ? (L.n + 255) / 256 : 128), dim3(256), 0, s, w.at<int>(L.total0),
                       w.at<int>(L.witness0), L.n, w.at<int>(L.slot_of), w.at<int>(L.count), w.at<int>(L.rank),
                       w.at<int>(L.witness), w.at<uint64_t>(L.fronts_slot), w.at<uint64_t>(L.fronts_orig), w.at<int>(L.fsize),
                       fill_dist ? w.at<float>(L.dist) : (float*)nullptr, w.ctrl(), w.at<SortParam>(L.sortparam));
    EVX_LAUNCH_CHECK();
    if (w.matrix_unless > 0) {  // the size of front 0 is known now: the matrix, if anybody is going to read it
      if (int e = dispatch_dominance_prefix(w, s, 2)) return e;
      w.matrix_unless = 0;
    }
  }
  return 0;
}

static int grant_dynamic_lds(const void* kernel, size_t lds);

// Resident blocks per CU of the peel kernel for a dynamic-LDS size (cached: the query is not free).
// Returns a negative library code or positive hipError_t through *err and 0 on failure.
static int peel_blocks_per_cu(size_t lds, int* err) {
  struct Entry { size_t lds; int dev; int per_cu; };
  static Entry cache[16];
  static int used = 0;
  static std::mutex mu;
  int dev = 0;
  (void)hipGetDevice(&dev);
  {
    std::lock_guard<std::mutex> lock(mu);
    for (int i = 0; i < used; ++i)
      if (cache[i].lds == lds && cache[i].dev == dev) return cache[i].per_cu;
  }
  if (int e = grant_dynamic_lds(reinterpret_cast<const void*>(peel_kernel), lds)) { *err = e; return 0; }
  int per_cu = 0;
  hipError_t e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, peel_kernel, kPeelThreads, lds);
  if (e != hipSuccess) { *err = (int)e; return 0; }
  if (per_cu < 1) { *err = kErrBadArg; return 0; }
  {
    std::lock_guard<std::mutex> lock(mu);
    if (used < 16) cache[used++] = Entry{lds, dev, per_cu};
  }
  return per_cu;
}

// Grants only ever grow per (kernel, device), and are made one at a time: a thread that was given a large size never
// finds it taken back by another thread's smaller one between its grant and its launch.
static int grant_dynamic_lds(const void* kernel, size_t lds) {
  if (lds > 160 * 1024) return kErrBadArg;  // (what a workgroup of this device can have)
  if (lds <= 48 * 1024) return 0;
  struct Entry { const void* kernel; int dev; size_t lds; };
  static Entry table[128];
  static int used = 0;
  static std::mutex mu;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) dev = -1;
  std::lock_guard<std::mutex> lock(mu);
  int at = -1;
  for (int i = 0; i < used; ++i)
    if (table[i].kernel == kernel && table[i].dev == dev) at = i;
  if (at >= 0 && table[at].lds >= lds) return 0;
  hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (e != hipSuccess) return (int)e;
  if (at >= 0)
    table[at].lds = lds;
  else if (used < 128)
    table[used++] = Entry{kernel, dev, lds};
  return 0;
}

// Sweeping workgroups of the LDS-resident peel for this population and the dynamic LDS each needs; 0 when the
// population does not fit (or the option is off).  Every workgroup takes a compute unit of its own.
constexpr size_t kLdsPeelBudget = 160 * 1024 - 512;

// Workgroups of peel_lds_kernel that a compute unit holds at once when each has `lds` bytes of dynamic LDS (asked of
// the runtime once per device and 8 KB step of the size, for the upper end of the step); 0 when the query fails.
static int lds_peel_per_cu(size_t lds) {
  static std::atomic<int> cache[64][24];  // 0 unknown, else the answer + 1
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64 || lds > kLdsPeelBudget) return 0;
  const int slot = (int)((lds + 8191) / 8192);
  int known = cache[dev][slot].load(std::memory_order_acquire);
  if (known == 0) {
    // (the attribute belongs to the (kernel, device) pair)
    // (both instances of the kernel: the one for several populations only moves its pointers first)
    int per_cu = 1 << 30;
    const size_t upper = (size_t)slot * 8192 < kLdsPeelBudget ? (size_t)slot * 8192 : kLdsPeelBudget;
    for (const void* kernel : {reinterpret_cast<const void*>(peel_lds_kernel<false>), reinterpret_cast<const void*>(peel_lds_kernel<true>)}) {
      if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLdsPeelBudget) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
      }
      int one = 0;
      if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&one, kernel, kLdsPeelThreads, upper) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
      }
      if (one < per_cu) per_cu = one;
    }
    known = per_cu + 1;
    cache[dev][slot].store(known, std::memory_order_release);
  }
  return known - 1;
}

// batch > 1: that many populations share the launch, each with this many sweeping workgroups (and its lister); up to
// four workgroups then share a compute unit where their LDS allows it, and the plan is the one with the most
// sweeping workgroups per population.
static int lds_peel_plan(const Layout& L, size_t* lds_out, int batch = 1) {
  if (!opt().peel_lds || L.n > 32768 || L.nwords > kLdsPeelThreads) return 0;  // (the lister keeps original indices in 16 bits and takes a bitmap word per thread)
  if (batch > 1) {
    size_t tail_need = opt().peel_tail ? peel_tail_lds_bytes(L.n, L.m) : 0;  // (a small last front is ordered in the kernel's LDS)
    if (tail_need > kLdsPeelBudget) tail_need = 0;
    int wanted = opt().peel_lds_blocks;
    if (wanted == 0) wanted = L.n / 64 < 32 ? 32 : L.n / 64;
    int best = 0;
    for (int per_cu = 1; per_cu <= 4; ++per_cu) {
      const int64_t share = (int64_t)per_cu * device_cus() / batch - 1;
      const int most = share < 255 ? (int)share : 255;
      if (most < 8) continue;
      const size_t limit = (size_t)160 * 1024 / per_cu - 1024;
      auto fits = [&](int sweepers) {
        const size_t b = lds_peel_bytes(L.n, L.nwords, sweepers);
        return b != 0 && b <= limit;
      };
      int sweepers = wanted < most ? wanted : most;
      while (sweepers < most && !fits(sweepers)) sweepers = sweepers + 8 < most ? sweepers + 8 : most;
      if (!fits(sweepers) || tail_need > limit || sweepers <= best) continue;
      const size_t lds = lds_peel_bytes(L.n, L.nwords, sweepers);
      if (lds_peel_per_cu(lds > tail_need ? lds : tail_need) < per_cu) continue;
      best = sweepers;
      *lds_out = lds;
    }
    return best;
  }
  const int most = device_cus() - 1 < 255 ? device_cus() - 1 : 255;  // + the lister; a record holds at least 4 units
  if (most < 8) return 0;
  auto fits = [&](int sweepers) {
    const size_t b = lds_peel_bytes(L.n, L.nwords, sweepers);
    return b != 0 && b <= kLdsPeelBudget;
  };
  if (!fits(most)) return 0;
  int sweepers = opt().peel_lds_blocks;
  if (sweepers == 0) {
    // by size: about 64 rows per workgroup, at least 32 workgroups
    sweepers = L.n / 64 < 32 ? 32 : L.n / 64;
  }
  if (sweepers > most) sweepers = most;
  while (sweepers < most && !fits(sweepers)) sweepers = sweepers + 8 < most ? sweepers + 8 : most;
  *lds_out = lds_peel_bytes(L.n, L.nwords, sweepers);
  return sweepers;
}

static int launch_lds_peel(const Ws& w, int64_t stop_count, bool want_perm, bool fill_dist, int sweepers, size_t lds, hipStream_t s,
                           bool order_last_front = false) {
  const Layout& L = w.L;
  if (stop_count < 1 || stop_count > L.n) return kErrBadArg;
  PeelTail tail;
  tail.mode = 0;
  tail.m = L.m;
  tail.npad = L.npad;
  tail.xs_sorted = w.at<float>(L.xs_sorted);
  tail.dist = w.at<float>(L.dist);
  tail.order = w.at<int>(L.order);
  tail.buffer = w.at<unsigned long long>(L.tailbuf);
  if (order_last_front && opt().peel_tail) {
    // a small last front is ordered by the peel kernel itself; its LDS must hold the candidates
    const size_t need = peel_tail_lds_bytes(L.n, L.m);
    if (need != 0 && need <= kLdsPeelBudget) {
      tail.mode = 2;
      if (lds < need) lds = need;
    }
  }
  // every workgroup waits for every other one, so the grid must be resident at once
  if ((int64_t)lds_peel_per_cu(lds) * device_cus() < (int64_t)(sweepers + 1) * w.batch) return kErrNotResident;
  auto launch = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, dim3(sweepers + 1, 1, w.batch), dim3(kLdsPeelThreads), lds, s, w.at<uint64_t>(L.dom), L.wstride, L.nwords, L.n,
                       w.at<int>(L.orig_of), w.at<int>(L.rank), fill_dist ? w.at<float>(L.dist) : (float*)nullptr,
                       w.at<uint64_t>(L.fronts_slot), w.at<uint64_t>(L.fronts_orig), w.at<int>(L.fsize),
                       want_perm ? w.at<int>(L.perm) : (int*)nullptr, w.at<int>(L.fstart), w.ctrl(), (int)stop_count, opt().spin_limit,
                       w.at<unsigned long long>(L.records), sweepers, tail, w.step);
  };
  if (w.batch > 1)
    launch(peel_lds_kernel<true>);
  else
    launch(peel_lds_kernel<false>);
  EVX_LAUNCH_CHECK();
  return 0;
}

// Counts and peeling for the entry points: one kernel when the matrix fits the LDS of the device, else the count
// pass over the matrix followed by a peel kernel that rescans rows in memory.
static int stage_peel(const Ws& w, int64_t stop_count, bool want_perm, hipStream_t s);
static int stage_count(const Ws& w, bool fill_dist, hipStream_t s, bool need_counts = true);
static int peel_pass_plan(const Layout& L, int* blocks_out, int* use_witness_out);
static int stage_peel_stepped(const Ws& w, int64_t stop_count, bool want_perm, hipStream_t s);
static int count_and_peel_persistent(const Ws& w, int64_t stop_count, bool want_perm, bool fill_dist, hipStream_t s,
                                     bool order_last_front, bool* may_have_ordered, bool* always_orders);

// used_stepped: the fronts were peeled one launch each (stepped.hpp) -- asked for by the tunable, or because the grids
// of the persistent kernels would not be resident at once on this device; the last front is then left to the caller.
static int count_and_peel(const Ws& w, int64_t stop_count, bool want_perm, bool fill_dist, hipStream_t s,
                          bool order_last_front = false, bool* may_have_ordered = nullptr, bool* always_orders = nullptr,
                          bool* used_stepped = nullptr) {
  if (used_stepped) *used_stepped = false;
  int e = kErrNotResident;
  if (!opt().peel_stepped) e = count_and_peel_persistent(w, stop_count, want_perm, fill_dist, s, order_last_front, may_have_ordered, always_orders);
  if (e != kErrNotResident) return e;
  if (may_have_ordered) *may_have_ordered = false;
  if (always_orders) *always_orders = false;
  if (used_stepped) *used_stepped = true;
  if (int c = stage_count(w, fill_dist, s, true)) return c;
  return stage_peel_stepped(w, stop_count, want_perm, s);
}

static int count_and_peel_persistent(const Ws& w, int64_t stop_count, bool want_perm, bool fill_dist, hipStream_t s,
                                     bool order_last_front, bool* may_have_ordered, bool* always_orders) {
  size_t lds = 0;
  if (may_have_ordered) *may_have_ordered = false;
  if (always_orders) *always_orders = false;
  if (const int sweepers = lds_peel_plan(w.L, &lds, w.batch)) {
    const bool may = order_last_front && opt().peel_tail && peel_tail_lds_bytes(w.L.n, w.L.m) != 0 &&
                     peel_tail_lds_bytes(w.L.n, w.L.m) <= kLdsPeelBudget;
    if (may_have_ordered) *may_have_ordered = may;
    if (always_orders && may) {
      // Whatever the last front turns out to be, the peel kernel orders it: no front of this population is too
      // large for it, and no workgroup can have more rows in one front than its record holds (a level with such a
      // record goes through the bitmaps in memory and leaves the last front to the kernels after it).
      int units = 2;
      while (units * 2 * sweepers <= kRecUnits && units < 32) units *= 2;
      const int waves = kLdsPeelThreads / 64;
      const int rows_of_a_workgroup = (w.L.n + sweepers * waves - 1) / (sweepers * waves) * waves;
      *always_orders = peel_tail_applies(w.L.n, w.L.m) && rows_of_a_workgroup <= 2 + 3 * (units - 1);
    }
    return launch_lds_peel(w, stop_count, want_perm, fill_dist, sweepers, lds, s, order_last_front);
  }
  if (w.batch > 1) return kErrNotResident;  // (the kernels below take one population per launch)
  // (the witness passes read of a row only its highest dominator: the count stage then walks every row from the top
  // as far as that, instead of adding up all of it)
  int blocks = 0, use_witness = 0;
  if (int e = peel_pass_plan(w.L, &blocks, &use_witness)) return e;
  if (int e = stage_count(w, fill_dist, s, use_witness == 0)) return e;
  return stage_peel(w, stop_count, want_perm, s);
}

// Grid of the peel kernels that rescan rows in memory, and whether they use the witness pass (else the sweep pass,
// which needs the popcounts of the rows).
static int peel_pass_plan(const Layout& L, int* blocks_out, int* use_witness_out) {
  const size_t lds_limit = 160 * 1024 - 4096;
  const size_t bitmap = sizeof(uint64_t) * (size_t)L.nwords;
  const int cus = device_cus();
  // The grid never exceeds what the device holds at once (the blocks wait for one another).
  auto grid_for = [&](size_t lds, int* err) -> int {
    int per_cu = peel_blocks_per_cu(lds, err);
    if (per_cu > opt().peel_blocks_per_cu) per_cu = opt().peel_blocks_per_cu;
    int64_t blocks = (int64_t)cus * per_cu;
    if (blocks > kMaxGrid) blocks = kMaxGrid;
    const int64_t wpb = kPeelThreads / 64;
    const int64_t useful = kFirstSweeper + ((int64_t)L.n + wpb - 1) / wpb;  // master, lister + one wave per row
    return (int)(blocks < useful ? blocks : useful);
  };
  // The witness pass keeps two bitmaps in LDS and at most kWitnessChunks * 64 rows per sweeping
  // wave; populations too large for that use the sweep pass.
  int err = 0;
  int use_witness = opt().peel_witness && 2 * bitmap <= lds_limit;
  int blocks = 0;
  if (use_witness) {
    blocks = grid_for(2 * bitmap, &err);
    if (err) return err;
    const int64_t waves = (int64_t)(blocks - kFirstSweeper) * (kPeelThreads / 64);
    if (blocks <= kFirstSweeper || (L.n + waves - 1) / waves > kWitnessChunks * 64) use_witness = 0;
  }
  if (!use_witness) {
    if (bitmap > lds_limit) return kErrBadArg;
    blocks = grid_for(bitmap, &err);
    if (err) return err;
  }
  if (blocks <= kFirstSweeper) return kErrNotResident;
  *blocks_out = blocks;
  *use_witness_out = use_witness;
  return 0;
}

static int stage_peel(const Ws& w, int64_t stop_count, bool want_perm, hipStream_t s) {
  const Layout& L = w.L;
  if (stop_count < 1 || stop_count > L.n) return kErrBadArg;
  const size_t bitmap = sizeof(uint64_t) * (size_t)L.nwords;
  const int cus = device_cus();
  int blocks = 0, use_witness = 0;
  if (int e = peel_pass_plan(L, &blocks, &use_witness)) return e;
  if (use_witness && opt().peel_records && L.n <= kRecordsMaxRowsWide) {
    // all-to-all records: 1 lister + a power of two of sweeping blocks, all resident at once
    // by size: 64 blocks up to 32768 rows, 128 above (measured at 20000 rows: 221 us per selection with 64
    // blocks, 225 with 128, 228 with 32, 238 with 192; between 1200 and 6000 rows the count hardly matters)
    const int by_size = L.n <= 32768 ? 64 : 128;
    const int sweepers = cus >= 64 ? (opt().peel_record_blocks ? opt().peel_record_blocks : by_size) : 16;
    const int wpb = kRecThreads / 64;
    const int list_capacity = wpb * ((L.n + sweepers * wpb - 1) / (sweepers * wpb));
    const size_t rec_lds = bitmap + 24 * (size_t)list_capacity;  // queue (8 + 4 + 4) and ranked pairs (2 x 4) per row
    // every block waits for every other one: all of them must be resident at once
    int rec_per_cu = 0;
    const bool wide = L.n > kRecordsMaxRows;
    const void* kernel = wide ? reinterpret_cast<const void*>(peel_records_kernel<true>)
                              : reinterpret_cast<const void*>(peel_records_kernel<false>);
    const bool rows_fit = (int64_t)list_capacity <= (int64_t)wpb * kWitnessChunks * 64;  // what the waves' registers hold
    if (rows_fit && rec_lds <= 150 * 1024)
      if (int e = grant_dynamic_lds(kernel, rec_lds)) return e;
    const hipError_t oe = wide ? hipOccupancyMaxActiveBlocksPerMultiprocessor(&rec_per_cu, peel_records_kernel<true>, kRecThreads, rec_lds)
                               : hipOccupancyMaxActiveBlocksPerMultiprocessor(&rec_per_cu, peel_records_kernel<false>, kRecThreads, rec_lds);
    if (oe != hipSuccess) return (int)oe;
    if (rows_fit && rec_lds <= 150 * 1024 && (int64_t)rec_per_cu * cus >= sweepers + 1) {
    hipLaunchKernelGGL(wide ? peel_records_kernel<true> : peel_records_kernel<false>, dim3(sweepers + 1), dim3(kRecThreads), rec_lds, s, w.at<uint64_t>(L.dom), L.wstride,
                       L.nwords, L.n, w.at<int>(L.orig_of), w.at<int>(L.rank), w.at<uint64_t>(L.fronts_slot),
                       w.at<uint64_t>(L.fronts_orig), w.at<int>(L.fsize), want_perm ? w.at<int>(L.perm) : (int*)nullptr,
                       w.at<int>(L.fstart), w.ctrl(), (int)stop_count, opt().spin_limit, w.at<int>(L.witness),
                       w.at<unsigned long long>(L.records), sweepers, list_capacity);
    EVX_LAUNCH_CHECK();
    return 0;
    }  // otherwise: the master protocol below, whose grid is sized to what fits
  }
  const size_t lds = bitmap * (use_witness ? 2 : 1);
  hipLaunchKernelGGL(peel_kernel, dim3(blocks), dim3(kPeelThreads), lds, s, w.at<uint64_t>(L.dom), L.wstride, L.nwords,
                     L.n, w.at<int>(L.orig_of), w.at<int>(L.count), w.at<int>(L.rank), w.at<uint64_t>(L.fronts_slot),
                     w.at<uint64_t>(L.fronts_orig), w.at<int>(L.fsize),
                     want_perm ? w.at<int>(L.perm) : (int*)nullptr, w.at<int>(L.fstart), w.ctrl(), (int)stop_count,
                     opt().spin_limit, w.at<int>(L.witness), use_witness);
  EVX_LAUNCH_CHECK();
  return 0;
}

// One launch per front, in groups; between groups the host waits for the stream and reads whether the pass that finds
// the ranking complete has run (the only place where this path waits).  stage_count must have left the full counts.
constexpr int kStepGroup = 16;
static int stage_peel_stepped(const Ws& w, int64_t stop_count, bool want_perm, hipStream_t s) {
  const Layout& L = w.L;
  if (stop_count < 1 || stop_count > L.n) return kErrBadArg;
  const size_t lds = sizeof(uint64_t) * (size_t)((L.nwords + 1) & ~1);
  if (int e = grant_dynamic_lds(reinterpret_cast<const void*>(step_pass_kernel), lds)) return e;
  int sweepers = (L.n + kStepThreads / 64 - 1) / (kStepThreads / 64);
  const int cap = device_cus() * 8;
  if (sweepers > cap) sweepers = cap;
  const int listers = (L.nwords + kStepListWords - 1) / kStepListWords;
  // (front L.n - 1 is the last that can exist; the pass after a front is the one that sees it complete)
  for (int64_t level = 1; level <= (int64_t)L.n + 1;) {
    for (int k = 0; k < kStepGroup && level <= (int64_t)L.n + 1; ++k, ++level) {
      hipLaunchKernelGGL(step_pass_kernel, dim3(sweepers + listers), dim3(kStepThreads), lds, s, w.at<uint64_t>(L.dom), L.wstride,
                         L.nwords, L.n, w.at<int>(L.orig_of), w.at<int>(L.count), w.at<int>(L.rank), w.at<uint64_t>(L.fronts_slot),
                         w.at<uint64_t>(L.fronts_orig), w.at<int>(L.fsize), w.at<int>(L.fstart),
                         want_perm ? w.at<int>(L.perm) : (int*)nullptr, w.ctrl(), (int)stop_count, (int)level, sweepers);
      EVX_LAUNCH_CHECK();
    }
    int32_t head[16];
    hipError_t e = hipMemcpyAsync(head, w.ctrl(), sizeof(head), hipMemcpyDeviceToHost, s);
    if (e != hipSuccess) return (int)e;
    e = hipStreamSynchronize(s);
    if (e != hipSuccess) return (int)e;
    static_assert(offsetof(Ctrl, reserved) == 40 && sizeof(int32_t) * (10 + kStepDone + 1) <= sizeof(head), "Ctrl.reserved[kStepDone]");
    if (head[0] != 0 || head[10 + kStepDone] != 0) break;
  }
  return 0;
}

static RadixBuffers radix_buffers(const Ws& w) {
  RadixBuffers b;
  b.pairs[0] = w.at<unsigned long long>(w.L.rpairs0);
  b.pairs[1] = w.at<unsigned long long>(w.L.rpairs1);
  b.table = w.at<int>(w.L.rtable);
  b.totals = w.at<int>(w.L.rtotals);
  b.kstride = w.L.kstride;
  return b;
}

// Blocks of a radix kernel: master + idle slot + one worker per 1024 candidates, all resident.
static int radix_grid(const Layout& L) {
  int workers = (L.n + 1023) / 1024;
  const int cap = device_cus() * 2 - kFirstSweeper;
  if (workers > cap) workers = cap;
  if (workers > kRadixMaxWorkers) workers = kRadixMaxWorkers;
  if (workers < 1) workers = 1;
  return workers + kFirstSweeper;
}

// Grid of the two kernels that order the last front (finish.hpp): the radix grid when a front of this
// population can exceed kRadixMinCandidates rows (they then synchronise across blocks), else one block
// per 256 candidates and objective.
// A last front of more than kMidSortMinCandidates rows in a population of at most kMidArgsortRows: its orders come from
// workgroups that sort in LDS without waiting for each other (finish.hpp), one per compute unit.
static bool crowd_mid_sort(const Layout& L) { return opt().mid_argsort != 0 && L.n > kMidSortMinCandidates && L.n <= kMidArgsortRows; }
// A larger population: such a front gets a launch of its own (its kernels have kMidArgsortThreads threads, the radix
// sort of a larger front kRadixThreads); each of the two returns at once from a front that is the other's.
static bool crowd_mid_split(const Layout& L) { return opt().mid_argsort != 0 && L.n > kMidArgsortRows; }

static int finish_grid(const Layout& L, int per_candidate_block) {
  if (crowd_mid_sort(L)) return device_cus();  // (their LDS leaves room for one workgroup per compute unit: all resident)
  if (L.n > kRadixMinCandidates) {
    // The kernels choose on the device: a front of at most kRadixMinCandidates rows is still ordered by counting,
    // one work item per 256 candidates (and objective), and wants as many blocks as it has items -- a population
    // of 5000 rows has a radix grid of 7 blocks, on which the 110 items of a 2764-row front of ten objectives took
    // 0.59 ms.  More workers than the radix sort needs only idle at its barriers.
    int blocks = radix_grid(L);
    int wanted = (kRadixMinCandidates / 256) * per_candidate_block + kFirstSweeper;
    int cap = device_cus() * 2;
    if (cap > kRadixMaxWorkers + kFirstSweeper) cap = kRadixMaxWorkers + kFirstSweeper;
    if (wanted > cap) wanted = cap;
    return blocks > wanted ? blocks : wanted;
  }
  int blocks = ((L.n + 255) / 256) * per_candidate_block;
  return blocks < 1 ? 1 : blocks;
}

// The grid of one population when `batch` of them share a launch whose workgroups may wait for each other: the device
// holds `resident` such workgroups at once.
static int shared_grid(int grid, int resident, int batch) {
  if (batch <= 1) return grid;
  const int cap = resident / batch < 1 ? 1 : resident / batch;
  return grid < cap ? grid : cap;
}

// phase 0: totals and matrix in one launch (or what the tunable prefix_mode asks for); 1: the totals alone, and the
// pairwise kernel for a population that is not finite; 2: the matrix alone, unless front 0 holds w.matrix_unless rows.
template <int M>
static int launch_dominance_prefix(const Ws& w, hipStream_t s, int phase) {
  constexpr int WW = M <= kPrefixWideObjectives ? 8 : 4;  // words per tile: what the LDS holds tables for
  // up to four objectives the tables of two tiles fit: a workgroup then builds whole 128-byte lines of the matrix
  constexpr int TT = M <= 4 ? 2 : 1;
  const Layout& L = w.L;
  const int shift = prefix_bucket_shift(L.n);
  const int buckets = ((L.n - 1) >> shift) + 1;
  const int bands_wanted = opt().prefix_bands;
  // bands of rows shared by all tiles (their stores then fall into the same rows at about the same time) pay from
  // about 100 000 rows on: 200 000 x 8 1203 -> 1156 us, 100 000 x 8 441 -> 424, but 65536 x 3 181 -> 190
  const int bands = bands_wanted != 0 && L.n >= 98304 ? 1 : 0;
  // shorter stretches for smaller populations, so that the workgroups still outnumber the compute units
  const int chunk = L.n >= 131072 ? kPrefixRowChunk : (L.n >= 65536 ? kPrefixRowChunk / 2 : kPrefixRowChunk / 4);
  const int stretches = (L.n + chunk - 1) / chunk;
  auto launch = [&](auto kernel, int tt) -> int {
    const size_t lds = (size_t)tt * prefix_lds_bytes(M, WW, buckets);
    if (int e = grant_dynamic_lds(reinterpret_cast<const void*>(kernel), lds)) return e;
    const int tiles = (int)round_up((L.nwords + WW * tt - 1) / (WW * tt), 128 / (WW * tt));
    hipLaunchKernelGGL(kernel, dim3(tiles, stretches), dim3(kPrefixThreads), lds, s, w.at<int>(L.pos), w.at<int>(L.scost),
                       w.at<uint32_t>(L.kid_sorted), w.at<uint64_t>(L.dom), L.n, L.kstride, L.wstride, L.nwords, shift, buckets,
                       chunk, bands, phase == 0 ? opt().prefix_mode : phase, w.at<int>(L.total0), w.at<int>(L.witness0),
                       w.at<SortParam>(L.sortparam), phase == 2 ? w.at<int>(L.fsize) : (const int*)nullptr, (int)w.matrix_unless);
    EVX_LAUNCH_CHECK();
    return 0;
  };
  // (200 000 x 3: 957 -> 769 us, x 4: 972 -> 797; 100 000 x 3: 319 -> 317; 65536 x 3: 184 -> 220: half as many workgroups)
  if (TT == 2 && opt().prefix_double_tile > 0 && L.n >= opt().prefix_double_tile) {
    if (int e = launch(dominance_prefix_kernel<M, WW, TT>, TT)) return e;
  } else {
    if (int e = launch(dominance_prefix_kernel<M, WW, 1>, 1)) return e;
  }
  if (phase == 2) return 0;
  // a population with a NaN or an infinity: the pairwise kernel, on a grid that costs nothing when it has nothing to do
  hipLaunchKernelGGL(dominance_nonfinite_kernel<M>, dim3(device_cus() * 8), dim3(256), 0, s, w.at<float>(L.xs_sorted),
                     w.at<uint64_t>(L.key_sorted), w.at<uint32_t>(L.kid_sorted), w.at<uint64_t>(L.dom), L.n, L.npad, L.wstride,
                     L.nwords, w.at<SortParam>(L.sortparam));
  EVX_LAUNCH_CHECK();
  return 0;
}

// The matrix of a large finite population from the order of its rows in every objective (prefix.hpp).  The
// buffers of the crowding stage (radix pairs, pos, scost) are free until then and carry the orders.
template <int M>
static int launch_dominance_prefix(const Ws& w, hipStream_t s, int phase);

static int stage_dominance_prefix(const Ws& w, bool orders_only, hipStream_t s, int64_t count_first) {
  const Layout& L = w.L;
  // (the count stage launches the second phase: the peel that keeps the matrix in LDS has no count stage)
  size_t unused = 0;
  const int phase = count_first > 0 && !orders_only && opt().prefix_count_first && opt().prefix_mode == 3 &&
                            lds_peel_plan(L, &unused, 1) == 0 ? 1 : 0;
  if (phase == 1) w.matrix_unless = count_first;
  if (L.n <= kMidArgsortRows && opt().mid_argsort) {
    // the orders from workgroups that sort in LDS: two launches, no grid barrier (and no barrier words to reset)
    const size_t sort_lds = mid_sort_lds_bytes(L.n);
    const bool wide = L.n <= kMidArgsortWideRows;
    const void* const kernel = wide ? reinterpret_cast<const void*>(objective_order_lds_kernel<true>)
                                    : reinterpret_cast<const void*>(objective_order_lds_kernel<false>);
    if (int e = grant_dynamic_lds(kernel, sort_lds)) return e;
    if (wide)
      hipLaunchKernelGGL(objective_order_lds_kernel<true>, dim3(device_cus()), dim3(kMidArgsortThreads), sort_lds, s, w.at<float>(L.xs),
                         L.npad, L.n, L.m, w.at<SortParam>(L.sortparam), w.ctrl(), w.at<int>(L.total0), w.at<int>(L.witness0),
                         radix_buffers(w));
    else
      hipLaunchKernelGGL(objective_order_lds_kernel<false>, dim3(device_cus()), dim3(kMidArgsortThreads), sort_lds, s, w.at<float>(L.xs),
                         L.npad, L.n, L.m, w.at<SortParam>(L.sortparam), w.ctrl(), w.at<int>(L.total0), w.at<int>(L.witness0),
                         radix_buffers(w));
    EVX_LAUNCH_CHECK();
    int64_t blocks = ((int64_t)L.n * L.m + 255) / 256;
    if (blocks > device_cus() * 8) blocks = device_cus() * 8;
    hipLaunchKernelGGL(objective_positions_kernel, dim3((unsigned)blocks), dim3(256), 0, s, L.n, L.m, w.at<int>(L.slot_of),
                       w.at<SortParam>(L.sortparam), w.ctrl(), w.at<int>(L.pos), w.at<int>(L.scost), radix_buffers(w));
    EVX_LAUNCH_CHECK();
    return orders_only ? 0 : dispatch_dominance_prefix(w, s, phase);
  }
  // shares of one objective's order that the streaming kernel would cut: as many as give every compute unit a
  // workgroup, if shares of kOrderStreamShare rows need no more than that
  const int stream_parts = device_cus() / L.m;
  if (opt().order_stream && L.n > kOrderStreamSample && L.n <= kOrderStreamMaxRows && (L.npad & 3) == 0 && stream_parts >= 1 &&
      stream_parts <= kOrderStreamSample && (int64_t)stream_parts * kOrderStreamShare >= L.n) {
    // larger populations likewise, by workgroups that read their objective's keys once and sort their share of the
    // order in LDS -- while those shares stay small: 40 000 x 8 the orders in 52 instead of 127 us, 65 536 x 3 57 / 90,
    // 100 000 x 8 105 / 144, 200 000 x 3 120 / 147; 200 000 x 8 (shares of 6250 rows) 201 / 185: the radix sort below
    const size_t stream_lds = sizeof(double) * kOrderStreamCapacity;
    if (int e = grant_dynamic_lds(reinterpret_cast<const void*>(objective_order_stream_kernel), stream_lds)) return e;
    const int parts = stream_parts;
    hipLaunchKernelGGL(objective_order_stream_kernel, dim3(L.m * parts), dim3(kOrderStreamThreads), stream_lds, s, w.at<float>(L.xs),
                       L.npad, L.n, L.m, parts, opt().order_stream_capacity, w.at<SortParam>(L.sortparam), w.ctrl(),
                       w.at<int>(L.total0), w.at<int>(L.witness0), radix_buffers(w));
    EVX_LAUNCH_CHECK();
    int64_t blocks = ((int64_t)L.n * L.m + 255) / 256;
    if (blocks > device_cus() * 8) blocks = device_cus() * 8;
    hipLaunchKernelGGL(objective_positions_kernel, dim3((unsigned)blocks), dim3(256), 0, s, L.n, L.m, w.at<int>(L.slot_of),
                       w.at<SortParam>(L.sortparam), w.ctrl(), w.at<int>(L.pos), w.at<int>(L.scost), radix_buffers(w));
    EVX_LAUNCH_CHECK();
    return orders_only ? 0 : dispatch_dominance_prefix(w, s, phase);
  }
  const size_t lds = kRadixLdsBytes;
  if (int e = grant_dynamic_lds(reinterpret_cast<const void*>(objective_order_kernel), lds)) return e;
  // more workers than one per 1024 rows: every one of them handles its share of all m segments
  int workers = (int)(((int64_t)L.n * L.m + 2047) / 2048);
  const int cap = (device_cus() * 2 < kRadixMaxWorkers + kFirstSweeper ? device_cus() * 2 : kRadixMaxWorkers + kFirstSweeper) - kFirstSweeper;
  if (workers > cap) workers = cap;
  if (workers + kFirstSweeper < radix_grid(L)) workers = radix_grid(L) - kFirstSweeper;
  hipLaunchKernelGGL(objective_order_kernel, dim3(workers + kFirstSweeper), dim3(kRadixThreads), lds, s, w.at<float>(L.xs), L.npad, L.n,
                     L.m, w.at<int>(L.slot_of), w.at<SortParam>(L.sortparam), w.ctrl(), w.at<int>(L.pos), w.at<int>(L.scost), w.at<int>(L.total0),
                     w.at<int>(L.witness0), radix_buffers(w), opt().spin_limit);
  EVX_LAUNCH_CHECK();
  // the barrier words of the control block restart from zero for the kernels that follow (the sort counted its
  // generations from a high base)
  const size_t first = offsetof(Ctrl, release);
  const int64_t words = (int64_t)((sizeof(Ctrl) + sizeof(unsigned long long) * kMaxGrid - first) / 4);
  hipLaunchKernelGGL(reset_state_kernel, dim3(16), dim3(256), 0, s, reinterpret_cast<uint32_t*>(w.base + L.ctrl + first), words);
  EVX_LAUNCH_CHECK();
  return orders_only ? 0 : dispatch_dominance_prefix(w, s, phase);
}

static int dispatch_dominance_prefix(const Ws& w, hipStream_t s, int phase) {
  switch (w.L.m) {
    case 2: return launch_dominance_prefix<2>(w, s, phase);
    case 3: return launch_dominance_prefix<3>(w, s, phase);
    case 4: return launch_dominance_prefix<4>(w, s, phase);
    case 5: return launch_dominance_prefix<5>(w, s, phase);
    case 6: return launch_dominance_prefix<6>(w, s, phase);
    case 7: return launch_dominance_prefix<7>(w, s, phase);
    case 8: return launch_dominance_prefix<8>(w, s, phase);
    case 9: return launch_dominance_prefix<9>(w, s, phase);
    case 10: return launch_dominance_prefix<10>(w, s, phase);
    case 11: return launch_dominance_prefix<11>(w, s, phase);
    case 12: return launch_dominance_prefix<12>(w, s, phase);
    case 13: return launch_dominance_prefix<13>(w, s, phase);
    case 14: return launch_dominance_prefix<14>(w, s, phase);
    case 15: return launch_dominance_prefix<15>(w, s, phase);
    case 16: return launch_dominance_prefix<16>(w, s, phase);
    default: return kErrBadArg;
  }
}

// Per-objective ordering of the candidates list[ctrl.worst_start ... + ctrl.nv).
// fused: 0 = the two kernels as stages of their own; 1 / 2 = a small front gets its distances (2: and the selection
// order) inside crowd_sort_kernel, and crowd_finish_kernel, given the same value, leaves it alone.
static CrowdArgs crowd_args(const Ws& w, const int* list, bool use_orders, int fused) {
  const Layout& L = w.L;
  CrowdArgs a;
  a.xs = w.at<float>(L.xs);
  a.npad = L.npad;
  a.list_base = list;
  a.ctrl = w.ctrl();
  a.m = L.m;
  a.kstride = L.kstride;
  a.pos = w.at<int>(L.pos);
  a.sorted_cost = w.at<float>(L.scost);
  a.buf = radix_buffers(w);
  a.spin_limit = opt().spin_limit;
  a.param = w.at<SortParam>(L.sortparam);
  a.use_orders = use_orders ? 1 : 0;
  a.fused = fused;
  a.mid_sort = crowd_mid_sort(L) ? 1 : (crowd_mid_split(L) ? 3 : 0);
  a.dist = w.at<float>(L.dist);
  a.dkey = w.at<uint32_t>(L.dkey);
  a.order = w.at<int>(L.order);
  a.ws_step = w.step;
  return a;
}

// The three launches that read the orders of a large last front off the orders of the whole population.
static int stage_front_orders(const Ws& w, const int* list, hipStream_t s) {
  const Layout& L = w.L;
  {
    const RadixBuffers b = radix_buffers(w);
    const int spans = (L.n + kFrontOrderSpan - 1) / kFrontOrderSpan;
    int* const number = reinterpret_cast<int*>(w.at<uint32_t>(L.dkey));  // free until the distances are known
    int* const per_span = b.table;
    hipLaunchKernelGGL(front_number_kernel, dim3((L.n + 1023) / 1024), dim3(256), 0, s, list, w.ctrl(),
                       w.at<SortParam>(L.sortparam), number);
    EVX_LAUNCH_CHECK();
    hipLaunchKernelGGL(front_order_count_kernel, dim3(spans, L.m), dim3(256), 0, s, b.pairs[0], b.kstride, L.n, w.at<int>(L.rank),
                       w.ctrl(), w.at<SortParam>(L.sortparam), per_span);
    EVX_LAUNCH_CHECK();
    hipLaunchKernelGGL(front_order_place_kernel, dim3(spans, L.m), dim3(256), 0, s, b.pairs[0], b.kstride, L.n,
                       w.at<int>(L.rank), w.ctrl(), w.at<SortParam>(L.sortparam), per_span, number, w.at<float>(L.xs), L.npad,
                       w.at<int>(L.pos), w.at<float>(L.scost));
    EVX_LAUNCH_CHECK();
  }
  return 0;
}

static size_t crowd_lds_bytes(const Layout& L, int fused) {
  size_t lds = sizeof(uint32_t) * kRadixMinCandidates + sizeof(uint64_t) * kRankTile;
  if (L.n > kRadixMinCandidates && kRadixLdsBytes > lds) lds = kRadixLdsBytes;
  if (fused != 0 && kFusedFrontLdsBytes > lds) lds = kFusedFrontLdsBytes;
  if (crowd_mid_sort(L) && mid_sort_lds_bytes(L.n) > lds) lds = mid_sort_lds_bytes(L.n);
  return lds;
}

static int stage_crowd_sort(const Ws& w, const int* list, bool use_orders, int fused, hipStream_t s, bool after_peel_tail = false) {
  const Layout& L = w.L;
  use_orders = use_orders && prefix_dominance_applies(L) && w.batch == 1;
  // a large front of a population whose matrix came from the per-objective orders: its own orders are read off
  // those (finish.hpp); the three kernels and the one below choose on the device which of them has work
  if (use_orders)
    if (int e = stage_front_orders(w, list, s)) return e;
  if (crowd_mid_split(L)) {
    const size_t mid_lds = mid_sort_lds_bytes(kMidArgsortRows);
    if (int e = grant_dynamic_lds(reinterpret_cast<const void*>(crowd_sort_kernel<kMidArgsortThreads, 2>), mid_lds)) return e;
    CrowdArgs a = crowd_args(w, list, use_orders, fused);
    a.mid_sort = 2;
    hipLaunchKernelGGL((crowd_sort_kernel<kMidArgsortThreads, 2>), dim3(device_cus()), dim3(kMidArgsortThreads), mid_lds, s, a,
                       after_peel_tail ? 1 : 0);
    EVX_LAUNCH_CHECK();
  }
  const size_t lds = crowd_lds_bytes(L, fused);
  const bool mid = crowd_mid_sort(L);
  const bool wide = L.n <= kMidArgsortWideRows;  // (which tables of the LDS sorter the population leaves room for)
  const bool many = w.batch > 1;
  auto instance = [&](auto one, auto several) { return many ? reinterpret_cast<const void*>(several) : reinterpret_cast<const void*>(one); };
  const void* const kernel = !mid   ? instance(crowd_sort_kernel<kRadixThreads, 0, false>, crowd_sort_kernel<kRadixThreads, 0, true>)
                             : wide ? instance(crowd_sort_kernel<kMidArgsortThreads, 1, false>, crowd_sort_kernel<kMidArgsortThreads, 1, true>)
                                    : instance(crowd_sort_kernel<kMidArgsortThreads, 2, false>, crowd_sort_kernel<kMidArgsortThreads, 2, true>);
  if (int e = grant_dynamic_lds(kernel, lds)) return e;
  // (the fused path ends with a barrier between all blocks: the grid must be resident at once, which a grid of at
  // most two blocks of 256 threads per compute unit is)
  int grid = finish_grid(L, L.m);
  if (fused != 0 && grid > device_cus() * 2) grid = device_cus() * 2;
  grid = shared_grid(grid, mid ? device_cus() : device_cus() * 2, w.batch);
  const CrowdArgs ca = crowd_args(w, list, use_orders, fused);
  const int tail_flag = after_peel_tail ? 1 : 0;
  if (mid && wide && many)
    hipLaunchKernelGGL((crowd_sort_kernel<kMidArgsortThreads, 1, true>), dim3(grid, 1, w.batch), dim3(kMidArgsortThreads), lds, s, ca, tail_flag);
  else if (mid && wide)
    hipLaunchKernelGGL((crowd_sort_kernel<kMidArgsortThreads, 1, false>), dim3(grid), dim3(kMidArgsortThreads), lds, s, ca, tail_flag);
  else if (mid && many)
    hipLaunchKernelGGL((crowd_sort_kernel<kMidArgsortThreads, 2, true>), dim3(grid, 1, w.batch), dim3(kMidArgsortThreads), lds, s, ca, tail_flag);
  else if (mid)
    hipLaunchKernelGGL((crowd_sort_kernel<kMidArgsortThreads, 2, false>), dim3(grid), dim3(kMidArgsortThreads), lds, s, ca, tail_flag);
  else if (many)
    hipLaunchKernelGGL((crowd_sort_kernel<kRadixThreads, 0, true>), dim3(grid, 1, w.batch), dim3(kRadixThreads), lds, s, ca, tail_flag);
  else
    hipLaunchKernelGGL((crowd_sort_kernel<kRadixThreads, 0, false>), dim3(grid), dim3(kRadixThreads), lds, s, ca, tail_flag);
  EVX_LAUNCH_CHECK();
  return 0;
}

// Crowding distances of those candidates and, with want_order, the selection order.
static int stage_crowd_finish(const Ws& w, const int* list, bool want_order, int fused, hipStream_t s, bool after_peel_tail = false) {
  const Layout& L = w.L;
  // (no front of this population is too large for the fused path of crowd_sort_kernel: nothing is left to do)
  if (fused != 0 && L.n <= kFusedFrontRows && (int64_t)L.n * L.m <= kFusedFrontValues && L.m <= kFusedFrontObjectives) return 0;
  if (crowd_mid_split(L)) {
    const size_t mid_lds = mid_sort_lds_bytes(kMidArgsortRows);
    if (int e = grant_dynamic_lds(reinterpret_cast<const void*>(crowd_finish_kernel<kMidArgsortThreads, 2>), mid_lds)) return e;
    CrowdArgs a = crowd_args(w, list, false, fused);
    a.mid_sort = 2;
    hipLaunchKernelGGL((crowd_finish_kernel<kMidArgsortThreads, 2>), dim3(device_cus()), dim3(kMidArgsortThreads), mid_lds, s, a,
                       want_order ? 1 : 0, after_peel_tail ? 1 : 0);
    EVX_LAUNCH_CHECK();
  }
  const size_t lds = crowd_lds_bytes(L, 0);
  const bool mid = crowd_mid_sort(L);
  const bool wide = L.n <= kMidArgsortWideRows;
  const bool many = w.batch > 1;
  auto instance = [&](auto one, auto several) { return many ? reinterpret_cast<const void*>(several) : reinterpret_cast<const void*>(one); };
  const void* const kernel = !mid   ? instance(crowd_finish_kernel<kRadixThreads, 0, false>, crowd_finish_kernel<kRadixThreads, 0, true>)
                             : wide ? instance(crowd_finish_kernel<kMidArgsortThreads, 1, false>, crowd_finish_kernel<kMidArgsortThreads, 1, true>)
                                    : instance(crowd_finish_kernel<kMidArgsortThreads, 2, false>, crowd_finish_kernel<kMidArgsortThreads, 2, true>);
  if (int e = grant_dynamic_lds(kernel, lds)) return e;
  const int grid = shared_grid(finish_grid(L, 1), mid ? device_cus() : device_cus() * 2, w.batch);
  const CrowdArgs ca = crowd_args(w, list, false, fused);
  const int order_flag = want_order ? 1 : 0, tail_flag = after_peel_tail ? 1 : 0;
  if (mid && wide && many)
    hipLaunchKernelGGL((crowd_finish_kernel<kMidArgsortThreads, 1, true>), dim3(grid, 1, w.batch), dim3(kMidArgsortThreads), lds, s, ca, order_flag, tail_flag);
  else if (mid && wide)
    hipLaunchKernelGGL((crowd_finish_kernel<kMidArgsortThreads, 1, false>), dim3(grid), dim3(kMidArgsortThreads), lds, s, ca, order_flag, tail_flag);
  else if (mid && many)
    hipLaunchKernelGGL((crowd_finish_kernel<kMidArgsortThreads, 2, true>), dim3(grid, 1, w.batch), dim3(kMidArgsortThreads), lds, s, ca, order_flag, tail_flag);
  else if (mid)
    hipLaunchKernelGGL((crowd_finish_kernel<kMidArgsortThreads, 2, false>), dim3(grid), dim3(kMidArgsortThreads), lds, s, ca, order_flag, tail_flag);
  else if (many)
    hipLaunchKernelGGL((crowd_finish_kernel<kRadixThreads, 0, true>), dim3(grid, 1, w.batch), dim3(kRadixThreads), lds, s, ca, order_flag, tail_flag);
  else
    hipLaunchKernelGGL((crowd_finish_kernel<kRadixThreads, 0, false>), dim3(grid), dim3(kRadixThreads), lds, s, ca, order_flag, tail_flag);
  EVX_LAUNCH_CHECK();
  return 0;
}

// The copy of a result of 4-byte elements out of the workspace, as the last kernel of an entry point: the result, or
// `poison` in every element when a device-side wait of the call ran out.
static int copy_out(const Ctrl* ctrl, void* dst, const void* src, int64_t n, uint32_t poison, hipStream_t s, int batch = 1,
                    int64_t ws_step = 0) {
  int64_t blocks = (n + 1023) / 1024;
  if (blocks > 1024) blocks = 1024;
  if (blocks < 1) blocks = 1;
  hipLaunchKernelGGL(copy_or_poison_kernel, dim3((unsigned)blocks, 1, batch), dim3(256), 0, s, ctrl, static_cast<const uint32_t*>(src),
                     static_cast<uint32_t*>(dst), n, poison, ws_step);
  EVX_LAUNCH_CHECK();
  return 0;
}
constexpr uint32_t kPoisonIndex = 0xFFFFFFFFu;  // -1 as a rank or an order
constexpr uint32_t kPoisonFloat = 0x7FC00000u;  // NaN as a distance

template <int M>
static int launch_batched_m(const BatchedArgs& a, int64_t batch, hipStream_t s) {
  const int nt = (int)round_up(a.n, 64);
  // (few populations of at most 256 rows: every workgroup has a compute unit, and every wave a SIMD, to itself -- 200 x 3:
  // the matrix in 7.5 instead of 12 us; with two waves to a SIMD the scalar loads win: 512 x 3 14 against 16.5 us)
  const bool stage = batch <= device_cus() && nt <= 256 && M <= 8 && opt().batched_stage;
  const size_t lds = batched_lds_bytes(nt, M) + (stage ? batched_stage_bytes(nt, M) : 0);
  // the attribute belongs to the (kernel, device) pair: remembered per device
  static size_t granted[64] = {0};
  static std::mutex mu;  // (a smaller grant by another thread must not follow a larger one)
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = -1;
  if (lds > 48 * 1024) {
    std::lock_guard<std::mutex> lock(mu);
    if (dev < 0 || lds > granted[dev]) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(batched_kernel<M>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      if (e != hipSuccess) return (int)e;
      if (dev >= 0) granted[dev] = lds;
    }
  }
  // grid.x carries the batch; very large batches go in slices
  for (int64_t b0 = 0; b0 < batch; b0 += 0x40000000ll) {
    BatchedArgs part = a;
    part.stage_fitness = stage ? 1 : 0;
    const int64_t nb = batch - b0 < 0x40000000ll ? batch - b0 : 0x40000000ll;
    part.f += b0 * a.f_stride_b;
    if (part.rank_all) part.rank_all += b0 * a.n;
    if (part.x) part.x += b0 * a.x_stride_b;
    if (part.out_x) part.out_x += b0 * a.stop_count * a.x_row_bytes;
    if (part.out_f) part.out_f += b0 * a.stop_count * a.m;
    if (part.out_rank) part.out_rank += b0 * a.stop_count;
    if (part.out_dist) part.out_dist += b0 * a.stop_count;
    hipLaunchKernelGGL(batched_kernel<M>, dim3((unsigned)nb), dim3(nt), lds, s, part);
    EVX_LAUNCH_CHECK();
  }
  return 0;
}

// Two objectives: one workgroup per population without a matrix (two_small.hpp), for up to kTwoSmallRows rows.
static int launch_two_small(const BatchedArgs& a, int64_t batch, hipStream_t s) {
  if (int e = grant_dynamic_lds(reinterpret_cast<const void*>(two_small_kernel), kTwoSmallLdsBytes)) return e;
  for (int64_t b0 = 0; b0 < batch; b0 += 0x40000000ll) {
    BatchedArgs part = a;
    const int64_t nb = batch - b0 < 0x40000000ll ? batch - b0 : 0x40000000ll;
    part.f += b0 * a.f_stride_b;
    if (part.rank_all) part.rank_all += b0 * a.n;
    if (part.x) part.x += b0 * a.x_stride_b;
    if (part.out_x) part.out_x += b0 * a.stop_count * a.x_row_bytes;
    if (part.out_f) part.out_f += b0 * a.stop_count * a.m;
    if (part.out_rank) part.out_rank += b0 * a.stop_count;
    if (part.out_dist) part.out_dist += b0 * a.stop_count;
    hipLaunchKernelGGL(two_small_kernel, dim3((unsigned)nb), dim3(kTwoSmallThreads), kTwoSmallLdsBytes, s, part);
    EVX_LAUNCH_CHECK();
  }
  return 0;
}

// Rows that the one-workgroup kernels take: the matrix kernel up to kBatchedMaxRows, two objectives up to kTwoSmallRows.
static int64_t batched_rows_limit(int64_t m) {
  if (m < 1 || m > kBatchedMaxObjectives) return 0;
  return m == 2 && opt().two_small_min_rows > 0 ? kTwoSmallRows : kBatchedMaxRows;
}

static int launch_batched(const BatchedArgs& a, int64_t batch, hipStream_t s) {
  if (a.m == 2 && opt().two_small_min_rows > 0 && (a.n >= opt().two_small_min_rows || a.n > kBatchedMaxRows))
    return launch_two_small(a, batch, s);
  switch (a.m) {
    case 1: return launch_batched_m<1>(a, batch, s);
    case 2: return launch_batched_m<2>(a, batch, s);
    case 3: return launch_batched_m<3>(a, batch, s);
    case 4: return launch_batched_m<4>(a, batch, s);
    case 5: return launch_batched_m<5>(a, batch, s);
    case 6: return launch_batched_m<6>(a, batch, s);
    case 7: return launch_batched_m<7>(a, batch, s);
    case 8: return launch_batched_m<8>(a, batch, s);
    case 9: return launch_batched_m<9>(a, batch, s);
    case 10: return launch_batched_m<10>(a, batch, s);
    case 11: return launch_batched_m<11>(a, batch, s);
    case 12: return launch_batched_m<12>(a, batch, s);
    case 13: return launch_batched_m<13>(a, batch, s);
    case 14: return launch_batched_m<14>(a, batch, s);
    case 15: return launch_batched_m<15>(a, batch, s);
    case 16: return launch_batched_m<16>(a, batch, s);
    default: return kErrBadArg;
  }
}

}  // namespace evx

using namespace evx;

static bool two_applies(const Layout& L, int64_t stop_count);
static int many_two_share(const Layout& L, int64_t batch, int64_t stop_count);
static int stage_rank_two(const Ws& w, const Fitness& src, int64_t stop_count, bool fill_dist, int* rank_until, hipStream_t s);

extern "C" {

int evox_hip_abi_version(void) { return EVOX_HIP_ABI_VERSION; }

size_t evox_hip_workspace_bytes(int64_t n, int64_t m) {
  Layout L;
  return make_layout(n, m, &L) ? L.total : 0;
}

int evox_hip_workspace_layout(int64_t n, int64_t m, int64_t* out) {
  Layout L;
  if (out == nullptr || !make_layout(n, m, &L)) return kErrBadArg;
  out[0] = (int64_t)L.dom;
  out[1] = L.wstride;
  out[2] = L.nwords;
  out[3] = (int64_t)L.count;
  out[4] = (int64_t)L.rank;
  out[5] = (int64_t)L.dist;
  out[6] = (int64_t)L.perm;
  out[7] = (int64_t)L.fstart;
  out[8] = (int64_t)L.order;
  out[9] = (int64_t)L.ctrl;
  out[10] = (int64_t)L.orig_of;
  return 0;
}

int evox_hip_slot_sort_layout(int64_t n, int64_t m, int64_t* out) {
  Layout L;
  if (out == nullptr || !make_layout(n, m, &L)) return kErrBadArg;
  out[0] = (int64_t)L.key_sorted;
  out[1] = (int64_t)L.kid_sorted;
  out[2] = (int64_t)L.xs_sorted;
  out[3] = (int64_t)L.xs;
  out[4] = L.npad;
  out[5] = (int64_t)L.slot_of;
  return 0;
}

static int set_named(Options& o, const char* name, int64_t value) {
  if (name == nullptr) return kErrBadArg;
  if (!strcmp(name, "peel_blocks_per_cu") && value >= 1 && value <= 16) {
    o.peel_blocks_per_cu = (int)value;
  } else if (!strcmp(name, "peel_witness") && (value == 0 || value == 1)) {
    o.peel_witness = (int)value;
  } else if (!strcmp(name, "peel_record_blocks") && (value == 0 || (value >= 16 && value <= 255))) {
    o.peel_record_blocks = (int)value;
  } else if (!strcmp(name, "peel_records") && (value == 0 || value == 1)) {
    o.peel_records = (int)value;
  } else if (!strcmp(name, "peel_lds") && (value == 0 || value == 1)) {
    o.peel_lds = (int)value;
  } else if (!strcmp(name, "tail_merged") && (value == 0 || value == 1)) {
    o.tail_merged = (int)value;
  } else if (!strcmp(name, "launch_memory") && (value == 0 || value == 1)) {
    o.launch_memory = (int)value;
  } else if (!strcmp(name, "peel_stepped") && (value == 0 || value == 1)) {
    o.peel_stepped = (int)value;
  } else if (!strcmp(name, "two_small_min_rows") && value >= 0) {
    o.two_small_min_rows = value;
  } else if (!strcmp(name, "two_min_rows") && value >= 0) {
    o.two_min_rows = value;
    if (value < o.two_min_rows_partial) o.two_min_rows_partial = value;  // (a lower limit asked for counts for both)
  } else if (!strcmp(name, "two_min_rows_partial") && value >= 0) {
    o.two_min_rows_partial = value;
  } else if (!strcmp(name, "peel_tail") && (value == 0 || value == 1)) {
    o.peel_tail = (int)value;
  } else if (!strcmp(name, "peel_lds_blocks") && (value == 0 || (value >= 8 && value <= 255))) {
    o.peel_lds_blocks = (int)value;
  } else if (!strcmp(name, "spin_limit") && value >= 1 && value <= 0x7FFFFFFFll) {
    o.spin_limit = (unsigned)value;
  } else if (!strcmp(name, "dominance_tile_words") && (value == 0 || value == 2 || value == 4 || value == 8 || value == 16)) {
    o.dominance_tile_words = (int)value;
  } else if (!strcmp(name, "dominance_folded") && (value == 0 || value == 1)) {
    o.dominance_folded = (int)value;
  } else if (!strcmp(name, "small_sort") && (value == 0 || value == 1)) {
    o.small_sort = (int)value;
  } else if (!strcmp(name, "mid_argsort") && (value == 0 || value == 1)) {
    o.mid_argsort = (int)value;
  } else if (!strcmp(name, "prefix_min_rows") && value >= 0) {
    o.prefix_min_rows = value;
  } else if (!strcmp(name, "prefix_double_tile") && value >= 0) {
    o.prefix_double_tile = value;
  } else if (!strcmp(name, "prefix_mode") && value >= 1 && value <= 3) {
    o.prefix_mode = (int)value;
  } else if (!strcmp(name, "prefix_bands") && (value == 0 || value == 1)) {
    o.prefix_bands = (int)value;
  } else if (!strcmp(name, "batched_stage") && (value == 0 || value == 1)) {
    o.batched_stage = (int)value;
  } else if (!strcmp(name, "order_stream") && (value == 0 || value == 1)) {
    o.order_stream = (int)value;
  } else if (!strcmp(name, "order_stream_capacity") && value >= 1 && value <= kOrderStreamCapacity) {
    o.order_stream_capacity = (int)value;
  } else if (!strcmp(name, "prefix_count_first") && (value == 0 || value == 1)) {
    o.prefix_count_first = (int)value;
  } else {
    return kErrBadArg;
  }
  return 0;
}

int evox_hip_set_option(const char* name, int64_t value) { return set_named(g_opt, name, value); }

struct evox_hip_options {
  evx::Options values;
};

evox_hip_options* evox_hip_options_create(void) {
  evox_hip_options* h = new (std::nothrow) evox_hip_options;
  if (h != nullptr) h->values = g_opt;
  return h;
}

void evox_hip_options_destroy(evox_hip_options* options) {
  if (options != nullptr && t_opt == &options->values) t_opt = nullptr;
  delete options;
}

int evox_hip_options_set(evox_hip_options* options, const char* name, int64_t value) {
  return options == nullptr ? kErrBadArg : set_named(options->values, name, value);
}

int evox_hip_options_use(const evox_hip_options* options) {
  t_opt = options == nullptr ? nullptr : &options->values;
  return 0;
}

int evox_hip_stage_prepare(const float* f, int64_t n, int64_t m, int64_t sr, int64_t sc, void* ws, size_t ws_bytes,
                           void* stream) {
  Ws w;
  if (int e = open_ws(n, m, ws, ws_bytes, &w)) return e;
  return stage_prepare(w, one_part(f, n, sr, sc), true, (hipStream_t)stream);
}

int evox_hip_stage_dominance(int64_t n, int64_t m, int variant, void* ws, size_t ws_bytes, void* stream) {
  Ws w;
  if (int e = open_ws(n, m, ws, ws_bytes, &w)) return e;
  return stage_dominance(w, variant, (hipStream_t)stream);
}

int evox_hip_stage_count(int64_t n, int64_t m, void* ws, size_t ws_bytes, void* stream) {
  Ws w;
  if (int e = open_ws(n, m, ws, ws_bytes, &w)) return e;
  // as a stage of its own it may be repeated on one dominance matrix: start from a clean state
  const int64_t zero_words = (int64_t)((w.L.zero_end - w.L.ctrl) / 4);
  int blocks = (int)((zero_words + 255) / 256);
  if (blocks > 1024) blocks = 1024;
  hipLaunchKernelGGL(reset_state_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, w.at<uint32_t>(w.L.ctrl), zero_words);
  EVX_LAUNCH_CHECK();
  return stage_count(w, true, (hipStream_t)stream);
}

int evox_hip_stage_peel(int64_t n, int64_t m, int64_t stop_count, int32_t* rank_out, void* ws, size_t ws_bytes,
                        void* stream) {
  Ws w;
  if (int e = open_ws(n, m, ws, ws_bytes, &w)) return e;
  // (the kernel that peels from LDS counts for itself; after stage_count it finds the same front 0 again.  As in the
  // selection it also orders a small last front: that part reads memory which stage_prepare clears, so a timing
  // of it repeats the stages from stage_prepare on)
  size_t lds = 0;
  if (const int sweepers = lds_peel_plan(w.L, &lds)) {
    if (int e = launch_lds_peel(w, stop_count, true, true, sweepers, lds, (hipStream_t)stream, true)) return e;
  } else if (int e = stage_peel(w, stop_count, true, (hipStream_t)stream)) {
    return e;
  }
  if (rank_out) return copy_out(w.ctrl(), rank_out, w.at<int>(w.L.rank), n, kPoisonIndex, (hipStream_t)stream);
  return 0;
}

int evox_hip_stage_crowding(int64_t n, int64_t m, void* ws, size_t ws_bytes, void* stream) {
  Ws w;
  if (int e = open_ws(n, m, ws, ws_bytes, &w)) return e;
  if (int e = stage_crowd_sort(w, w.at<int>(w.L.perm), true, 0, (hipStream_t)stream)) return e;
  return stage_crowd_finish(w, w.at<int>(w.L.perm), false, 0, (hipStream_t)stream);
}

int evox_hip_stage_order(int64_t n, int64_t m, void* ws, size_t ws_bytes, void* stream) {
  Ws w;
  if (int e = open_ws(n, m, ws, ws_bytes, &w)) return e;
  return stage_crowd_finish(w, w.at<int>(w.L.perm), true, 0, (hipStream_t)stream);
}

}  // extern "C"

// batch > 1: that many populations of one shape in the same launches (see select_rows); their ranks lie n elements apart.
static int rank_rows(const Fitness& fit, int64_t n, int64_t m, int64_t stop_count, int32_t* rank_out, void* ws, size_t ws_bytes,
                     hipStream_t s, int batch = 1, int64_t ws_step = 0) {
  Ws w;
  if (rank_out == nullptr || stop_count < 1 || stop_count > n) return kErrBadArg;
  if (int e = open_ws(n, m, ws, ws_bytes, &w)) return e;
  if (batch > 1) {
    if (ws_step < (int64_t)w.L.total || (ws_step & 255) != 0 || ws_bytes < (size_t)ws_step * (size_t)batch) return kErrWorkspace;
    w.batch = batch;
    w.step = ws_step;
  }
  if (batch == 1 ? two_applies(w.L, stop_count) : many_two_share(w.L, batch, stop_count) >= batch) {
    int* until = stop_count < n ? w.at<int>(w.L.order) : (int*)nullptr;
    const int e = stage_rank_two(w, fit, stop_count, false, until, s);
    if (e != kErrNotResident || batch > 1) {
      if (e) return e == kErrNotResident ? kErrBadArg : e;
      return copy_out(w.ctrl(), rank_out, until != nullptr ? until : w.at<int>(w.L.rank), n, kPoisonIndex, s, w.batch, w.step);
    }
  }
  if (int e = stage_prepare(w, fit, true, s)) return e;
  if (int e = stage_dominance(w, kDomAuto, s)) return e;
  if (batch > 1) {
    if (int e = count_and_peel_persistent(w, stop_count, false, false, s, false, nullptr, nullptr)) return e == kErrNotResident ? kErrBadArg : e;
  } else if (int e = count_and_peel(w, stop_count, false, false, s)) {
    return e;
  }
  return copy_out(w.ctrl(), rank_out, w.at<int>(w.L.rank), n, kPoisonIndex, s, w.batch, w.step);
}

extern "C" {

int evox_hip_non_dominate_rank_until(const float* f, int64_t n, int64_t m, int64_t sr, int64_t sc, int64_t stop_count,
                                     int32_t* rank_out, void* ws, size_t ws_bytes, void* stream) {
  return rank_rows(one_part(f, n, sr, sc), n, m, stop_count, rank_out, ws, ws_bytes, (hipStream_t)stream);
}

int evox_hip_non_dominate_rank(const float* f, int64_t n, int64_t m, int64_t sr, int64_t sc, int32_t* rank_out, void* ws,
                               size_t ws_bytes, void* stream) {
  return evox_hip_non_dominate_rank_until(f, n, m, sr, sc, n, rank_out, ws, ws_bytes, stream);
}

size_t evox_hip_first_front_workspace_bytes(int64_t n, int64_t m) {
  Layout L;
  return make_layout(n, m, &L) ? L.dom : 0;
}

}  // extern "C"

// batch > 1: that many populations of one shape in the same launches, their workspaces (without the matrix) ws_step
// bytes apart, their masks n bytes.
static int first_front_rows(const Fitness& fit, int64_t n, int64_t m, uint8_t* mask_out, void* ws, size_t ws_bytes, hipStream_t s,
                            int batch = 1, int64_t ws_step = 0) {
  Ws w;
  if (mask_out == nullptr) return kErrBadArg;
  if (int e = open_ws(n, m, ws, ws_bytes, &w, false)) return e;
  const Layout& L = w.L;
  if (batch > 1) {
    if (ws_step < (int64_t)L.dom || (ws_step & 255) != 0 || ws_bytes < (size_t)ws_step * (size_t)batch) return kErrWorkspace;
    w.batch = batch;
    w.step = ws_step;
  }
  if (int e = stage_prepare(w, fit, true, s)) return e;
  switch (L.m) {
    case 1: launch_first_front<1>(w, mask_out, s); break;
    case 2: launch_first_front<2>(w, mask_out, s); break;
    case 3: launch_first_front<3>(w, mask_out, s); break;
    case 4: launch_first_front<4>(w, mask_out, s); break;
    case 5: launch_first_front<5>(w, mask_out, s); break;
    case 6: launch_first_front<6>(w, mask_out, s); break;
    case 7: launch_first_front<7>(w, mask_out, s); break;
    case 8: launch_first_front<8>(w, mask_out, s); break;
    case 9: launch_first_front<9>(w, mask_out, s); break;
    case 10: launch_first_front<10>(w, mask_out, s); break;
    case 11: launch_first_front<11>(w, mask_out, s); break;
    case 12: launch_first_front<12>(w, mask_out, s); break;
    case 13: launch_first_front<13>(w, mask_out, s); break;
    case 14: launch_first_front<14>(w, mask_out, s); break;
    case 15: launch_first_front<15>(w, mask_out, s); break;
    case 16: launch_first_front<16>(w, mask_out, s); break;
    default:
      hipLaunchKernelGGL(first_front_any_m_kernel, dim3((L.n + 255) / 256, 1, w.batch), dim3(256), 0, s, w.at<float>(L.xs_sorted),
                         w.at<uint32_t>(L.kid_sorted), w.at<int>(L.orig_of), L.n, L.npad, L.m, mask_out, w.ctrl(), w.step);
  }
  EVX_LAUNCH_CHECK();
  return 0;
}

// batch > 1: as above; the masks lie mask_step bytes apart, the distances n elements.
static int crowding_rows(const Fitness& costs, int64_t n, int64_t m, const uint8_t* mask, int64_t mask_stride, int64_t mask_step,
                         float* dist_out, void* ws, size_t ws_bytes, hipStream_t s, int batch = 1, int64_t ws_step = 0) {
  Ws w;
  if (costs.f == nullptr || dist_out == nullptr) return kErrBadArg;
  if (int e = open_ws(n, m, ws, ws_bytes, &w, batch == 1)) return e;
  const Layout& L = w.L;
  if (batch > 1) {
    if (ws_step < (int64_t)L.dom || (ws_step & 255) != 0 || ws_bytes < (size_t)ws_step * (size_t)batch) return kErrWorkspace;
    w.batch = batch;
    w.step = ws_step;
  }
  if (int e = stage_prepare(w, costs, false, s)) return e;
  hipLaunchKernelGGL(compact_mask_kernel, dim3(1, 1, w.batch), dim3(1024), 0, s, mask, mask_stride, L.n, w.at<int>(L.perm),
                     w.at<float>(L.dist), w.ctrl(), mask_step, w.step);
  EVX_LAUNCH_CHECK();
  if (int e = stage_crowd_sort(w, w.at<int>(L.perm), false, 1, s)) return e;
  if (int e = stage_crowd_finish(w, w.at<int>(L.perm), false, 1, s)) return e;
  return copy_out(w.ctrl(), dist_out, w.at<float>(L.dist), n, kPoisonFloat, s, w.batch, w.step);
}

// Populations that share the launches of a first-front mask or of the crowding distances: their kernels need no
// matrix, so a copy of the workspace is small; as many as 1 GiB of workspace holds (for the crowding distances:
// and as the kernels that order a front, whose workgroups wait for each other, can be resident together).
static int many_small_share(const Layout& L, int64_t batch, bool crowding) {
  if (batch < 2) return 1;
  if (crowding && (L.n > kMidArgsortRows || (!opt().mid_argsort && L.n > kRadixMinCandidates))) return 1;
  int64_t share = (int64_t)(1ull << 30) / (int64_t)align_up(L.dom);
  if (crowding && share > device_cus() / 2) share = device_cus() / 2;
  if (share > 32768) share = 32768;
  if (share > batch) share = batch;
  if (share < 2) return 1;
  const int64_t passes = (batch + share - 1) / share;
  return (int)((batch + passes - 1) / passes);
}

extern "C" {

int evox_hip_first_front_mask(const float* f, int64_t n, int64_t m, int64_t sr, int64_t sc, uint8_t* mask_out, void* ws,
                              size_t ws_bytes, void* stream) {
  return first_front_rows(one_part(f, n, sr, sc), n, m, mask_out, ws, ws_bytes, (hipStream_t)stream);
}

size_t evox_hip_many_first_front_workspace_bytes(int64_t batch, int64_t n, int64_t m) {
  Layout L;
  if (batch < 1 || !make_layout(n, m, &L)) return 0;
  return align_up(L.dom) * (size_t)many_small_share(L, batch, false);
}

int evox_hip_many_first_front_mask(const float* f, int64_t batch, int64_t n, int64_t m, int64_t stride_batch, int64_t sr, int64_t sc,
                                   uint8_t* mask_out, void* ws, size_t ws_bytes, void* stream) {
  Layout L;
  if (f == nullptr || mask_out == nullptr || batch < 1 || !make_layout(n, m, &L)) return kErrBadArg;
  const int share = many_small_share(L, batch, false);
  for (int64_t b0 = 0; b0 < batch;) {
    const int64_t left = batch - b0;
    const int count = (int)(left < share ? left : share);
    if (int e = first_front_rows(one_part(f + b0 * stride_batch, n, sr, sc, stride_batch), n, m, mask_out + b0 * n, ws, ws_bytes,
                                 (hipStream_t)stream, count, count > 1 ? (int64_t)align_up(L.dom) : 0))
      return e;
    b0 += count;
  }
  return 0;
}

size_t evox_hip_many_crowding_workspace_bytes(int64_t batch, int64_t n, int64_t m) {
  Layout L;
  if (batch < 1 || !make_layout(n, m, &L)) return 0;
  const int share = many_small_share(L, batch, true);
  return share > 1 ? align_up(L.dom) * (size_t)share : L.total;
}

int evox_hip_many_crowding_distance(const float* costs, int64_t batch, int64_t n, int64_t m, int64_t stride_batch, int64_t sr,
                                    int64_t sc, const uint8_t* mask, int64_t mask_batch_stride, int64_t mask_stride, float* dist_out,
                                    void* ws, size_t ws_bytes, void* stream) {
  Layout L;
  if (costs == nullptr || dist_out == nullptr || batch < 1 || !make_layout(n, m, &L)) return kErrBadArg;
  const int share = many_small_share(L, batch, true);
  for (int64_t b0 = 0; b0 < batch;) {
    const int64_t left = batch - b0;
    const int count = (int)(left < share ? left : share);
    if (int e = crowding_rows(one_part(costs + b0 * stride_batch, n, sr, sc, stride_batch), n, m,
                              mask != nullptr ? mask + b0 * mask_batch_stride : nullptr, mask_stride, mask_batch_stride,
                              dist_out + b0 * n, ws, ws_bytes, (hipStream_t)stream, count, count > 1 ? (int64_t)align_up(L.dom) : 0))
      return e;
    b0 += count;
  }
  return 0;
}

int evox_hip_crowding_distance(const float* costs, int64_t n, int64_t m, int64_t sr, int64_t sc, const uint8_t* mask,
                               int64_t mask_stride, float* dist_out, void* ws, size_t ws_bytes, void* stream) {
  if (costs == nullptr) return kErrBadArg;
  return crowding_rows(one_part(costs, n, sr, sc), n, m, mask, mask_stride, 0, dist_out, ws, ws_bytes, (hipStream_t)stream);
}

}  // extern "C"

// Workspace of the standalone stable argsort: control block with barrier slots, two pair buffers, the
// per-block digit table and the digit totals.
struct SortLayout {
  int n, kstride, workers;
  size_t ctrl, pairs0, pairs1, table, totals, total;
};

static bool make_sort_layout(int64_t n, SortLayout* L) {
  if (n < 1 || n > 0x7FFFFF00ll) return false;
  L->n = (int)n;
  L->kstride = (int)round_up(n, 64);
  int workers = (int)((n + 1023) / 1024);
  if (workers > kRadixMaxWorkers) workers = kRadixMaxWorkers;
  L->workers = workers;
  size_t o = 0;
  L->ctrl = o;    o = align_up(o + sizeof(Ctrl) + sizeof(unsigned long long) * kMaxGrid);
  L->pairs0 = o;  o = align_up(o + sizeof(unsigned long long) * (size_t)L->kstride);
  L->pairs1 = o;  o = align_up(o + sizeof(unsigned long long) * (size_t)L->kstride);
  L->table = o;   o = align_up(o + sizeof(int) * 256 * (size_t)kRadixMaxWorkers);
  L->totals = o;  o = align_up(o + sizeof(int) * 256);
  L->total = o;
  return true;
}

// key_cap: see argsort_step_kernel (device memory or null; only the sort of more than kMidArgsortRows keys looks at it).
static int argsort_step(const void* key, int kind, int64_t stride, int64_t n, const int32_t* prev_order, int32_t* order_out,
                        void* ws, size_t ws_bytes, void* stream, const int* key_cap = nullptr) {
  SortLayout L;
  if (key == nullptr || order_out == nullptr || kind < 0 || kind > 2) return kErrBadArg;
  if (!make_sort_layout(n, &L)) return kErrBadArg;
  if (ws == nullptr || ws_bytes < L.total || (reinterpret_cast<uintptr_t>(ws) & 255u) != 0) return kErrWorkspace;
  hipStream_t s = (hipStream_t)stream;
  if (n <= kSmallArgsortRows) {
    const int npad = ((int)n + 127) & ~127;
    if (int e = grant_dynamic_lds(reinterpret_cast<const void*>(small_argsort_kernel), sizeof(double) * (size_t)npad)) return e;
    hipLaunchKernelGGL(small_argsort_kernel, dim3(npad / kSmallArgsortGroup), dim3(kSmallArgsortThreads),
                       sizeof(double) * (size_t)npad, s, key, kind, stride, (int)n, prev_order, order_out);
    EVX_LAUNCH_CHECK();
    return 0;
  }
  if (n <= kMidArgsortRows && opt().mid_argsort) {
    // (one workgroup per compute unit, each producing a run of slots; no workgroup waits for another)
    const size_t lds = mid_sort_lds_bytes((int)n);
    const bool wide = n <= kMidArgsortWideRows;
    if (int e = grant_dynamic_lds(wide ? reinterpret_cast<const void*>(mid_argsort_kernel<true>)
                                       : reinterpret_cast<const void*>(mid_argsort_kernel<false>), lds))
      return e;
    const int per = (int)round_up((n + device_cus() - 1) / device_cus(), 16);
    if (wide)
      hipLaunchKernelGGL(mid_argsort_kernel<true>, dim3((unsigned)((n + per - 1) / per)), dim3(kMidArgsortThreads), lds, s, key, kind,
                         stride, (int)n, prev_order, per, order_out);
    else
      hipLaunchKernelGGL(mid_argsort_kernel<false>, dim3((unsigned)((n + per - 1) / per)), dim3(kMidArgsortThreads), lds, s, key, kind,
                         stride, (int)n, prev_order, per, order_out);
    EVX_LAUNCH_CHECK();
    return 0;
  }
  uint8_t* base = static_cast<uint8_t*>(ws);
  // every call starts from a cleared control block: barrier generations restart
  const int64_t zero_words = (int64_t)((L.pairs0 - L.ctrl) / 4);
  hipLaunchKernelGGL(reset_state_kernel, dim3(16), dim3(256), 0, s, reinterpret_cast<uint32_t*>(base + L.ctrl), zero_words);
  EVX_LAUNCH_CHECK();
  RadixBuffers b;
  b.pairs[0] = reinterpret_cast<unsigned long long*>(base + L.pairs0);
  b.pairs[1] = reinterpret_cast<unsigned long long*>(base + L.pairs1);
  b.table = reinterpret_cast<int*>(base + L.table);
  b.totals = reinterpret_cast<int*>(base + L.totals);
  b.kstride = L.kstride;
  int workers = L.workers;
  const int cap = device_cus() * 2 - kFirstSweeper;  // all blocks resident at once
  if (workers > cap) workers = cap;
  if (workers < 1) workers = 1;
  hipLaunchKernelGGL(argsort_step_kernel, dim3(workers + kFirstSweeper), dim3(kRadixThreads), kRadixLdsBytes, s, key, kind,
                     stride, L.n, prev_order, reinterpret_cast<Ctrl*>(base + L.ctrl), b, order_out, opt().spin_limit, key_cap);
  EVX_LAUNCH_CHECK();
  // (an order of -1 everywhere when one of the sort's grid barriers ran out)
  return copy_out(reinterpret_cast<const Ctrl*>(base + L.ctrl), order_out, nullptr, n, kPoisonIndex, s);
}

// One stable argsort step of int32 keys for each of `batch` populations in one launch (n <= kMidArgsortRows, the
// kernels that never wait): keys key_step bytes apart, orders order_step bytes apart.
static int argsort_step_many(const void* key, int64_t n, int batch, int64_t key_step, int32_t* order_out, int64_t order_step,
                             hipStream_t s) {
  if (n <= kSmallArgsortRows) {
    const int npad = ((int)n + 127) & ~127;
    if (int e = grant_dynamic_lds(reinterpret_cast<const void*>(small_argsort_kernel), sizeof(double) * (size_t)npad)) return e;
    hipLaunchKernelGGL(small_argsort_kernel, dim3(npad / kSmallArgsortGroup, batch), dim3(kSmallArgsortThreads),
                       sizeof(double) * (size_t)npad, s, key, (int)kKeyInt32, (int64_t)1, (int)n, (const int*)nullptr, order_out, key_step,
                       order_step);
    EVX_LAUNCH_CHECK();
    return 0;
  }
  if (n > kMidArgsortRows) return kErrBadArg;
  const size_t lds = mid_sort_lds_bytes((int)n);
  const bool wide = n <= kMidArgsortWideRows;
  if (int e = grant_dynamic_lds(wide ? reinterpret_cast<const void*>(mid_argsort_kernel<true>)
                                     : reinterpret_cast<const void*>(mid_argsort_kernel<false>), lds))
    return e;
  // (a population's share of the compute units, at least sixteen workgroups)
  int blocks = device_cus() / batch;
  if (blocks < 16) blocks = 16;
  const int per = (int)round_up((n + blocks - 1) / blocks, 16);
  const dim3 grid((unsigned)((n + per - 1) / per), (unsigned)batch);
  if (wide)
    hipLaunchKernelGGL(mid_argsort_kernel<true>, grid, dim3(kMidArgsortThreads), lds, s, key, (int)kKeyInt32, (int64_t)1, (int)n,
                       (const int*)nullptr, per, order_out, key_step, order_step);
  else
    hipLaunchKernelGGL(mid_argsort_kernel<false>, grid, dim3(kMidArgsortThreads), lds, s, key, (int)kKeyInt32, (int64_t)1, (int)n,
                       (const int*)nullptr, per, order_out, key_step, order_step);
  EVX_LAUNCH_CHECK();
  return 0;
}

// `batch` sorts of n <= kSmallArgsortRows positions in one launch: a workgroup per sort, or several sorts per
// workgroup when they are short.
template <int T, int R>
static int launch_rows_argsort(const void* key, int kind, int64_t batch_stride, int64_t stride, int64_t batch, int n,
                               const int32_t* prev_order, int32_t* order_out, hipStream_t s) {
  int group = 1;
  while (group * R < n) group <<= 1;  // threads per sort, a power of two
  if (group > T) return kErrBadArg;
  const int rows_per_block = T / group;
  const int row_stride = rows_per_block > 1 ? (n | 1) : n;
  const size_t lds = sizeof(double) * (size_t)rows_per_block * (size_t)row_stride;
  if (int e = grant_dynamic_lds(reinterpret_cast<const void*>(rows_argsort_kernel<T, R>), lds)) return e;
  int64_t blocks = (batch + rows_per_block - 1) / rows_per_block;
  if (blocks > 65536) blocks = 65536;
  hipLaunchKernelGGL((rows_argsort_kernel<T, R>), dim3((unsigned)blocks), dim3(T), lds, s, key, kind, batch_stride, stride, batch, n,
                     rows_per_block, row_stride, prev_order, order_out);
  EVX_LAUNCH_CHECK();
  return 0;
}

static int launch_rows_bitonic(const void* key, int kind, int64_t batch_stride, int64_t stride, int64_t batch, int n,
                               const int32_t* prev_order, int32_t* order_out, hipStream_t s) {
  int npad = kRowsBitonicMin;
  while (npad < n) npad <<= 1;
  if (npad > kRowsArgsortMax) return kErrBadArg;
  const int threads = npad / 8 < 1024 ? npad / 8 : 1024;  // eight entries per thread and pass
  const size_t lds = sizeof(double) * (size_t)npad;
  if (int e = grant_dynamic_lds(reinterpret_cast<const void*>(rows_bitonic_argsort_kernel), lds)) return e;
  const int64_t blocks = batch < 65536 ? batch : 65536;
  hipLaunchKernelGGL(rows_bitonic_argsort_kernel, dim3((unsigned)blocks), dim3(threads), lds, s, key, kind, batch_stride, stride,
                     batch, n, npad, prev_order, order_out);
  EVX_LAUNCH_CHECK();
  return 0;
}

extern "C" {

size_t evox_hip_argsort_workspace_bytes(int64_t n) {
  SortLayout L;
  return make_sort_layout(n, &L) ? L.total : 0;
}

int evox_hip_stable_argsort_step(const void* key, int kind, int64_t stride, int64_t n, const int32_t* prev_order,
                                 int32_t* order_out, void* ws, size_t ws_bytes, void* stream) {
  return argsort_step(key, kind, stride, n, prev_order, order_out, ws, ws_bytes, stream);
}

int evox_hip_stable_argsort_step_batched(const void* key, int kind, int64_t batch_stride, int64_t stride, int64_t batch,
                                         int64_t n, const int32_t* prev_order, int32_t* order_out, void* ws, size_t ws_bytes,
                                         void* stream) {
  SortLayout L;
  if (key == nullptr || order_out == nullptr || kind < 0 || kind > 2 || batch < 1) return kErrBadArg;
  if (!make_sort_layout(n, &L)) return kErrBadArg;
  if (ws == nullptr || ws_bytes < L.total || (reinterpret_cast<uintptr_t>(ws) & 255u) != 0) return kErrWorkspace;
  hipStream_t s = (hipStream_t)stream;
  // all sorts in one launch when a sort fits the LDS of a workgroup: by counting up to 256 positions (several
  // sorts per workgroup), through a bitonic network above that
  if (batch >= 2 && n <= kRowsArgsortMax) {
    if (n <= 256) return launch_rows_argsort<256, 1>(key, kind, batch_stride, stride, batch, (int)n, prev_order, order_out, s);
    return launch_rows_bitonic(key, kind, batch_stride, stride, batch, (int)n, prev_order, order_out, s);
  }
  const size_t key_bytes = 4;
  for (int64_t b = 0; b < batch; ++b) {
    const void* kb = static_cast<const uint8_t*>(key) + (size_t)(b * batch_stride) * key_bytes;
    if (int e = argsort_step(kb, kind, stride, n, prev_order ? prev_order + b * n : nullptr, order_out + b * n, ws, ws_bytes, stream))
      return e;
  }
  return 0;
}

}  // extern "C"

// ---- fitness of 8-byte elements (wide.hpp)
struct WideLayout {
  int n, m;
  size_t ctrl, key_lo, key_hi, key_mask, selected, boundary, ord_a, ord_b, terms, dist, neg_lo, neg_hi, order_a, order_b, front_dkey,
      front_ends, sort_ws, sort_bytes, total;
};

static bool make_wide_layout(int64_t n, int64_t m, WideLayout* L) {
  if (n < 1 || m < 1 || n > 0x7FFFFF00ll || m > 65535 || n * m > 0x7FFFFFFFll * 16) return false;
  L->n = (int)n;
  L->m = (int)m;
  const size_t nm = (size_t)n * (size_t)m;
  size_t o = 0;
  L->ctrl = o;      o = align_up(o + sizeof(WideCtrl));
  L->key_lo = o;    o = align_up(o + 4 * nm);
  L->key_hi = o;    o = align_up(o + 4 * nm);
  L->key_mask = o;  o = align_up(o + 4 * (size_t)n);
  L->selected = o;  o = align_up(o + (size_t)n);
  L->boundary = o;  o = align_up(o + 4 * (size_t)n);
  L->ord_a = o;     o = align_up(o + 4 * nm);
  L->ord_b = o;     o = align_up(o + 4 * nm);
  L->terms = o;     o = align_up(o + 8 * nm);
  L->dist = o;      o = align_up(o + 8 * (size_t)n);
  L->neg_lo = o;    o = align_up(o + 4 * (size_t)n);
  L->neg_hi = o;    o = align_up(o + 4 * (size_t)n);
  L->order_a = o;   o = align_up(o + 4 * (size_t)n);
  L->order_b = o;   o = align_up(o + 4 * (size_t)n);
  L->front_dkey = o; o = align_up(o + 8 * (size_t)n);
  L->front_ends = o; o = align_up(o + 8 * (size_t)m);
  SortLayout sort_layout;
  if (!make_sort_layout(n, &sort_layout)) return false;
  L->sort_bytes = sort_layout.total;
  L->sort_ws = o;   o = align_up(o + L->sort_bytes);
  L->total = o;
  return true;
}

static int wide_grid(int64_t items) {
  int64_t blocks = (items + 255) / 256;
  const int64_t cap = (int64_t)device_cus() * 8;
  if (blocks > cap) blocks = cap;
  return (int)(blocks < 1 ? 1 : blocks);
}

// The crowding distances of the rows selected by the mask, by the rank vector (rank == its largest set value) or all
// rows, into `dist` (double for out_kind 0, float for 1), and with neg_keys the sort keys of their negatives.
static int wide_distances(const WideLayout& L, uint8_t* base, const void* costs, int kind, int64_t sr, int64_t sc,
                          const uint8_t* mask, int64_t mask_stride, const int32_t* rank, void* dist, int out_kind, bool neg_keys,
                          hipStream_t s, int* outcome = nullptr) {
  const int n = L.n, m = L.m;
  WideCtrl* ctrl = reinterpret_cast<WideCtrl*>(base + L.ctrl);
  uint32_t* key_lo = reinterpret_cast<uint32_t*>(base + L.key_lo);
  uint32_t* key_hi = reinterpret_cast<uint32_t*>(base + L.key_hi);
  int* key_mask = reinterpret_cast<int*>(base + L.key_mask);
  uint8_t* selected = base + L.selected;
  int* boundary = reinterpret_cast<int*>(base + L.boundary);
  int* ord_a = reinterpret_cast<int*>(base + L.ord_a);
  int* ord_b = reinterpret_cast<int*>(base + L.ord_b);
  hipLaunchKernelGGL(wide_head_kernel, dim3(1), dim3(1024), 0, s, mask, mask_stride, rank, n, ctrl);
  EVX_LAUNCH_CHECK();
  hipLaunchKernelGGL(wide_keys_kernel, dim3(wide_grid((int64_t)n * m)), dim3(256), 0, s, costs, kind, sr, sc, n, m, mask, mask_stride,
                     rank, ctrl, key_lo, key_hi, key_mask, selected, boundary);
  EVX_LAUNCH_CHECK();
  // per objective: by cost (low half, then high half of its ordered image), then selected rows first; ties by row
  void* sort_ws = base + L.sort_ws;
  if (int e = evox_hip_stable_argsort_step_batched(key_lo, kKeyUint32, n, 1, m, n, nullptr, ord_a, sort_ws, L.sort_bytes, s)) return e;
  if (int e = evox_hip_stable_argsort_step_batched(key_hi, kKeyUint32, n, 1, m, n, ord_a, ord_b, sort_ws, L.sort_bytes, s)) return e;
  const int* order = ord_b;
  if (mask != nullptr || rank != nullptr) {
    if (int e = evox_hip_stable_argsort_step_batched(key_mask, kKeyInt32, 0, 1, m, n, ord_b, ord_a, sort_ws, L.sort_bytes, s)) return e;
    order = ord_a;
  }
  uint32_t* neg_lo = neg_keys ? reinterpret_cast<uint32_t*>(base + L.neg_lo) : nullptr;
  uint32_t* neg_hi = neg_keys ? reinterpret_cast<uint32_t*>(base + L.neg_hi) : nullptr;
  if (out_kind == 0) {
    double* terms = reinterpret_cast<double*>(base + L.terms);
    hipLaunchKernelGGL(wide_terms_kernel<double>, dim3(wide_grid((int64_t)n * m)), dim3(256), 0, s, costs, kind, sr, sc, n, m, order, ctrl,
                       terms, boundary);
    EVX_LAUNCH_CHECK();
    hipLaunchKernelGGL(wide_sum_kernel<double>, dim3(wide_grid(n)), dim3(256), 0, s, terms, selected, boundary, ctrl, n, m,
                       static_cast<double*>(dist), neg_lo, neg_hi, outcome);
  } else {
    float* terms = reinterpret_cast<float*>(base + L.terms);
    hipLaunchKernelGGL(wide_terms_kernel<float>, dim3(wide_grid((int64_t)n * m)), dim3(256), 0, s, costs, kind, sr, sc, n, m, order, ctrl,
                       terms, boundary);
    EVX_LAUNCH_CHECK();
    hipLaunchKernelGGL(wide_sum_kernel<float>, dim3(wide_grid(n)), dim3(256), 0, s, terms, selected, boundary, ctrl, n, m,
                       static_cast<float*>(dist), neg_lo, neg_hi, outcome);
  }
  EVX_LAUNCH_CHECK();
  return 0;
}

// Whether the selection of a population of n rows orders its last front without sorting the costs
// (wide_select_direct): up to kWideDirectRows rows, unless the last selection of this shape found a front of more
// than kWideDirectFront rows -- that path's work grows with the square of the front.
static bool wide_direct_applies(int64_t n, const int* outcome) {
  return n <= kWideDirectRows && (outcome == nullptr || __atomic_load_n(outcome, __ATOMIC_RELAXED) != 2);
}

// The distances of the rows of the last front (rank == the largest rank set) and the selection order of all rows by
// (rank, distance descending, row index), for populations of up to kWideDirectRows rows: one stable argsort step of
// the ranks lists the rows, the kernels of wide.hpp do the rest without sorting the costs.
static int wide_select_direct(const WideLayout& L, uint8_t* base, const void* costs, int kind, int64_t sr, int64_t sc,
                              const int32_t* rank, void* dist, int out_kind, int* order_out, hipStream_t s, int* outcome,
                              int batch = 1, int64_t ws_step = 0, int64_t cost_step = 0) {
  // batch > 1: that many populations in the same launches, their workspaces ws_step bytes, their costs cost_step bytes and
  // their rank vectors n entries apart (dist and order_out lie in the workspaces)
  const int n = L.n, m = L.m;
  WideCtrl* ctrl = reinterpret_cast<WideCtrl*>(base + L.ctrl);
  int* listing = reinterpret_cast<int*>(base + L.order_b);
  uint64_t* key = reinterpret_cast<uint64_t*>(base + L.terms);
  uint64_t* dkey = reinterpret_cast<uint64_t*>(base + L.front_dkey);
  int* ends = reinterpret_cast<int*>(base + L.front_ends);
  hipLaunchKernelGGL(wide_head_kernel, dim3(1, 1, batch), dim3(1024), 0, s, (const uint8_t*)nullptr, (int64_t)0, rank, n, ctrl, ws_step);
  EVX_LAUNCH_CHECK();
  if (batch > 1) {
    if (int e = argsort_step_many(rank, n, batch, (int64_t)n * 4, listing, ws_step, s)) return e;
  } else if (int e = evox_hip_stable_argsort_step(rank, kKeyInt32, 1, n, nullptr, listing, base + L.sort_ws, L.sort_bytes, s)) {
    return e;
  }
  // (sixteen lanes per candidate; the grids are sized for a front of all rows, which the kernels find out on the device)
  const int pair_grid = shared_grid(wide_grid((int64_t)n * 16), device_cus() * 8, batch);
  const int keys_grid = shared_grid(wide_grid((int64_t)n * m), device_cus() * 8, batch);
  const int dist_grid = (n + 15) / 16;  // (a group of lanes per row, n <= kWideDirectRows)
  auto launch = [&](auto* typed_dist) {
    using Out = std::remove_pointer_t<decltype(typed_dist)>;
    hipLaunchKernelGGL(wide_front_keys_kernel<Out>, dim3(keys_grid < m ? m : keys_grid, 1, batch), dim3(256), 0, s, costs, kind, sr, sc, n,
                       m, listing, ctrl, key, ends, typed_dist, ws_step, cost_step);
    hipLaunchKernelGGL(wide_front_dist_kernel<Out>, dim3(dist_grid, 1, batch), dim3(256), 0, s, costs, kind, sr, sc, n, m, listing, ctrl,
                       key, ends, typed_dist, dkey, ws_step, cost_step);
  };
  if (out_kind == 0)
    launch(static_cast<double*>(dist));
  else
    launch(static_cast<float*>(dist));
  EVX_LAUNCH_CHECK();
  hipLaunchKernelGGL(wide_front_order_kernel, dim3(pair_grid, 1, batch), dim3(256), 0, s, listing, ctrl, dkey, n, order_out, outcome, ws_step);
  EVX_LAUNCH_CHECK();
  return 0;
}

// The gathers of a selection by `order` in one launch: x (if any), the fitness rows, the ranks and the distances.
struct WideGather {
  const void* x;
  int64_t x_row_bytes, x_row_stride_bytes, x_step;
  const void* f_rows;
  int64_t f_row_bytes, f_row_stride_bytes, f_step;
  const int32_t* rank;
  const void* dist;
  int64_t dist_bytes, dist_step;
  void *out_x, *out_f, *out_rank, *out_dist;
};
static int wide_gather(const WideGather& a, const int* order, int64_t order_step, int64_t n, int64_t topk, int batch, hipStream_t s) {
  GatherParts parts;
  parts.parts = 0;
  parts.first[0] = 0;
  auto add_part = [&](const void* src, int64_t row_bytes, int64_t row_stride_bytes, int64_t src_step, void* dst) {
    if (row_bytes <= 0) return;
    uintptr_t bits = reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst) | (uintptr_t)row_bytes | (uintptr_t)row_stride_bytes;
    if (batch > 1) bits |= (uintptr_t)src_step | (uintptr_t)(topk * row_bytes);
    const int unit = bits % 16 == 0 ? 16 : bits % 8 == 0 ? 8 : bits % 4 == 0 ? 4 : 1;
    const int p = parts.parts++;
    parts.src[p] = static_cast<const uint8_t*>(src);
    parts.dst[p] = static_cast<uint8_t*>(dst);
    parts.row_bytes[p] = row_bytes;
    parts.row_stride_bytes[p] = row_stride_bytes;
    parts.src_step[p] = src_step;
    parts.dst_step[p] = topk * row_bytes;
    parts.unit[p] = unit;
    parts.first[p + 1] = parts.first[p] + topk * (row_bytes / unit);
  };
  if (a.x != nullptr) add_part(a.x, a.x_row_bytes, a.x_row_stride_bytes, a.x_step, a.out_x);
  add_part(a.f_rows, a.f_row_bytes, a.f_row_stride_bytes, a.f_step, a.out_f);
  add_part(a.rank, 4, 4, n * 4, a.out_rank);
  add_part(a.dist, a.dist_bytes, a.dist_bytes, a.dist_step, a.out_dist);
  const int grid = shared_grid(wide_grid(parts.first[parts.parts]), device_cus() * 8, batch);
  hipLaunchKernelGGL(gather_parts_kernel, dim3(grid, 1, batch), dim3(256), 0, s, parts, order, topk, order_step);
  EVX_LAUNCH_CHECK();
  return 0;
}

namespace evx {
static size_t wide_workspace_need(int64_t n, int64_t m) {
  WideLayout L;
  return make_wide_layout(n, m, &L) ? L.total : 0;
}
}  // namespace evx

// Two objectives without a matrix (two.hpp): the rows sorted by (f1, f2, index), the fronts as rounds of prefix
// minima handed from workgroup to workgroup, the listing by (rank, index) from one stable argsort of the ranks.
static bool two_applies(const Layout& L, int64_t stop_count) {
  const int64_t least = stop_count >= L.n ? opt().two_min_rows : (opt().two_min_rows_partial > opt().two_min_rows ? opt().two_min_rows_partial : opt().two_min_rows);
  return L.m == 2 && opt().two_min_rows > 0 && L.n >= least && L.n <= kTwoMaxRows && !opt().peel_stepped;
}

// Several populations at once take that path when their argsort of the ranks is one of the kernels that never wait
// and all their chains are resident together: how many of `batch` share a launch (0: none).
static int many_two_share(const Layout& L, int64_t batch, int64_t stop_count) {
  if (batch < 2 || !two_applies(L, stop_count) || L.n > kMidArgsortRows || !opt().mid_argsort) return 0;
  const int blocks = (L.n + kTwoChunk - 1) / kTwoChunk;
  int share = device_cus() * 2 / blocks;
  if (share > batch) share = (int)batch;
  if (share < 2) return 0;
  const int64_t passes = (batch + share - 1) / share;
  return (int)((batch + passes - 1) / passes);
}

// Leaves what count_and_peel leaves: ranks by original index (of every row), the listing, the front starts and sizes
// and the control block's description of the front that holds the stop_count-th row.  rank_until: optionally the
// ranks with the rows behind that front unset (n ints).
static int stage_rank_two(const Ws& w, const Fitness& src, int64_t stop_count, bool fill_dist, int* rank_until, hipStream_t s) {
  const Layout& L = w.L;
  if (stop_count < 1 || stop_count > L.n) return kErrBadArg;
  WideLayout WL;
  if (!make_wide_layout(L.n, L.m, &WL) || WL.total > L.wide_bytes) return kErrWorkspace;
  if (int e = stage_prepare(w, src, true, s, true)) return e;
  const int blocks = (L.n + kTwoChunk - 1) / kTwoChunk;
  // (every workgroup waits for the one before it: resident at once on any device with as many compute units)
  if ((int64_t)blocks * w.batch > device_cus() * 2) return kErrNotResident;
  const float* xs_sorted = w.at<float>(L.xs_sorted);
  hipLaunchKernelGGL(two_peel_kernel, dim3(blocks, 1, w.batch), dim3(kTwoThreads), 0, s, xs_sorted, xs_sorted + L.npad,
                     w.at<uint32_t>(L.kid_sorted), w.at<int>(L.orig_of), L.n, w.at<int>(L.rank),
                     fill_dist ? w.at<float>(L.dist) : (float*)nullptr, w.ctrl(), w.at<unsigned long long>(L.two_ring), opt().spin_limit,
                     (int)stop_count, w.step);
  EVX_LAUNCH_CHECK();
  int grid = (L.n + 255) / 256;
  if (grid > device_cus() * 8) grid = device_cus() * 8;
  grid = shared_grid(grid, device_cus() * 8, w.batch);
  hipLaunchKernelGGL(two_finish_kernel, dim3(grid, 1, w.batch), dim3(256), 0, s, w.at<uint32_t>(L.kid_sorted), w.at<int>(L.orig_of),
                     xs_sorted, xs_sorted + L.npad, L.n, w.at<int>(L.rank), w.ctrl(), w.step);
  EVX_LAUNCH_CHECK();
  if (w.batch > 1) {
    if (int e = argsort_step_many(w.at<int>(L.rank), L.n, w.batch, w.step, w.at<int>(L.perm), w.step, s)) return e;
  } else {
    uint8_t* wb = w.base + L.wide;
    if (int e = argsort_step(w.at<int>(L.rank), kKeyInt32, 1, L.n, nullptr, w.at<int>(L.perm), wb + WL.sort_ws, WL.sort_bytes, s,
                             &w.ctrl()->reserved[kTwoRounds]))
      return e;
  }
  hipLaunchKernelGGL(two_bounds_kernel, dim3(grid, 1, w.batch), dim3(256), 0, s, w.at<int>(L.perm), w.at<int>(L.rank), L.n,
                     w.at<int>(L.fstart), w.ctrl(), (int)stop_count, w.step);
  EVX_LAUNCH_CHECK();
  hipLaunchKernelGGL(two_sizes_kernel, dim3(grid, 1, w.batch), dim3(256), 0, s, w.at<int>(L.perm), w.at<int>(L.rank), L.n,
                     w.at<int>(L.fstart), w.at<int>(L.fsize), w.ctrl(), rank_until, w.step);
  EVX_LAUNCH_CHECK();
  return 0;
}

// Shared body of the two selection entry points: the population is one part or two.
static int select_rows(const void* x, int64_t x_row_bytes, int64_t x_row_stride_bytes, const void* x2,
                       int64_t x2_row_stride_bytes, const Fitness& fit, int64_t n, int64_t m, int64_t topk, void* out_x,
                       float* out_f, int32_t* out_rank, float* out_dist, int32_t* out_order, void* ws, size_t ws_bytes,
                       hipStream_t s, bool may_allocate, int batch = 1, int64_t ws_step = 0, int64_t x_step_bytes = 0,
                       int64_t x2_step_bytes = 0) {
  // batch > 1: that many populations of one shape in the same launches (the caller has checked that their grids are
  // resident together: many_populations_plan); their workspaces lie ws_step bytes apart, their decision vectors
  // x_step_bytes, their fitness fit.step elements, their results topk rows
  Ws w;
  if (out_f == nullptr || out_rank == nullptr || out_dist == nullptr) return kErrBadArg;
  if ((x == nullptr) != (out_x == nullptr) || (x == nullptr) != (x2 == nullptr)) return kErrBadArg;
  if (x != nullptr && (x_row_bytes < 0 || x_row_stride_bytes < 0 || x2_row_stride_bytes < 0)) return kErrBadArg;
  if (topk < 1 || topk > n) return kErrBadArg;
  if (int e = open_ws(n, m, ws, ws_bytes, &w)) return e;
  const Layout& L = w.L;
  if (batch > 1) {
    if (ws_step < (int64_t)L.total || (ws_step & 255) != 0 || ws_bytes < (size_t)ws_step * (size_t)batch) return kErrWorkspace;
    w.batch = batch;
    w.step = ws_step;
  }
  int unit = 1;
  if (x != nullptr) {
    const uintptr_t bits = reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(x2) | reinterpret_cast<uintptr_t>(out_x) |
                           (uintptr_t)x_row_bytes | (uintptr_t)x_row_stride_bytes | (uintptr_t)x2_row_stride_bytes |
                           (uintptr_t)x_step_bytes | (uintptr_t)x2_step_bytes;
    unit = (bits % 16 == 0) ? 16 : (bits % 4 == 0) ? 4 : 1;
  }
  GatherArgs g = {};
  g.order = w.at<int>(L.order);
  g.listed = w.at<int>(L.perm);
  g.topk = (int)topk;
  g.x = static_cast<const uint8_t*>(x);
  g.x_row_stride = x_row_stride_bytes;
  g.x_row_bytes = x_row_bytes;
  g.out_x = static_cast<uint8_t*>(out_x);
  g.unit = unit;
  g.f = fit.f;
  g.f_stride_row = fit.sr;
  g.f_stride_col = fit.sc;
  g.n_first = (int)fit.n_first;
  g.x2 = static_cast<const uint8_t*>(x2);
  g.x2_row_stride = x2_row_stride_bytes;
  g.f2 = fit.f2;
  g.f2_stride_row = fit.sr2;
  g.f2_stride_col = fit.sc2;
  g.m = L.m;
  g.out_f = out_f;
  g.rank = w.at<int>(L.rank);
  g.out_rank = out_rank;
  g.dist = w.at<float>(L.dist);
  g.out_dist = out_dist;
  g.out_order = out_order;
  g.ctrl = w.ctrl();
  g.ws_step = w.step;
  g.x_step = x_step_bytes;
  g.x2_step = x2_step_bytes;
  g.f_step = fit.step;
  g.f2_step = fit.step2;
  int gather_blocks = (int)((topk + 3) / 4);
  if (gather_blocks > device_cus() * 8) gather_blocks = device_cus() * 8;
  const dim3 gather_grid(gather_blocks, 1, w.batch);
  auto launch_gather = [&](bool after_peel) {
    if (after_peel && w.batch > 1)
      hipLaunchKernelGGL(gather_after_peel_kernel<true>, gather_grid, dim3(256), 0, s, g);
    else if (after_peel)
      hipLaunchKernelGGL(gather_after_peel_kernel<false>, gather_grid, dim3(256), 0, s, g);
    else if (w.batch > 1)
      hipLaunchKernelGGL(gather_kernel<true>, gather_grid, dim3(256), 0, s, g);
    else
      hipLaunchKernelGGL(gather_kernel<false>, gather_grid, dim3(256), 0, s, g);
  };
  if (batch == 1 ? two_applies(L, topk) : many_two_share(L, batch, topk) >= batch) {
    const int e = stage_rank_two(w, fit, topk, true, nullptr, s);
    if (e != kErrNotResident || batch > 1) {
      if (e) return e == kErrNotResident ? kErrBadArg : e;
      // the last front by the ordering kernels, then the gather, as after a peel that leaves the last front alone
      if (int c = stage_crowd_sort(w, w.at<int>(L.perm), false, 2, s, false)) return c;
      if (int c = stage_crowd_finish(w, w.at<int>(L.perm), true, 2, s, false)) return c;
      launch_gather(false);
      EVX_LAUNCH_CHECK();
      return 0;
    }
  }
  if (int e = stage_prepare(w, fit, true, s)) return e;
  // A population that keeps filling what is kept from front 0 alone (many objectives, or converged) has no use for
  // the matrix: where the order-based kernel would build it, the word of the launch memory says what the last two
  // selections of the shape found, and the kernel counts first when both had enough in front 0 (200 000 x 8, half
  // kept: the stage 0.98 -> 0.80 ms; a wrong guess costs a second launch, 0.92 ms, once).
  int64_t count_first = 0;
  if (batch == 1 && opt().launch_memory && opt().prefix_count_first && prefix_dominance_applies(L) && !opt().peel_stepped) {
    g.front0_note = outcome_slot(n, m, may_allocate, s, 2);
    g.front0_size = w.at<int>(L.fsize);
    g.front0_enough = (int)topk;
    if (g.front0_note != nullptr && __atomic_load_n(g.front0_note, __ATOMIC_RELAXED) == 3) count_first = topk;
  }
  if (int e = stage_dominance(w, kDomAuto, s, count_first)) return e;
  bool peel_orders = false;  // the peel kernel orders a small last front itself (it says so in Ctrl.tail_done)
  bool peel_always_orders = false;  // ... and here every front is small enough: nothing is left to launch but the gather
  bool stepped = false;  // the fronts were peeled one launch each: the last front is ordered likewise, by the kernels of wide.hpp
  if (batch > 1) {
    if (int e = count_and_peel_persistent(w, topk, true, true, s, true, &peel_orders, &peel_always_orders)) return e == kErrNotResident ? kErrBadArg : e;
  } else if (int e = count_and_peel(w, topk, true, true, s, true, &peel_orders, &peel_always_orders, &stepped)) {
    return e;
  }
  g.order_from_peel = peel_always_orders ? 1 : 0;
  g.outcome = batch == 1 && peel_orders && !peel_always_orders && opt().launch_memory ? outcome_slot(n, m, may_allocate, s) : nullptr;
  const int last_outcome = g.outcome != nullptr ? __atomic_load_n(g.outcome, __ATOMIC_RELAXED) : 0;
  // Where the peel kernel may have ordered the last front, the kernels that would order it look at Ctrl.tail_done and
  // return at once.  A launch that does nothing still costs about 4.7 us, so with up to three objectives -- last
  // fronts of a few hundred rows, which the peel kernel orders -- the two ordering stages and the gather share one
  // launch (crowd_gather_kernel); with more objectives the last front is usually too large for the peel kernel, and
  // the two stages as kernels of their own, each on the grid that suits it, order it faster than the shared launch does
  // (20 000 x 5, a front of 2532 rows: 245 against 261 us per selection; 20 000 x 8, 7481 rows: 457 against 493).
  // What the last selection of this shape found decides where it is known: a population that has converged keeps
  // last fronts of thousands of rows, which the kernels of their own order 20-30 us faster (20 000 x 3, one front: 166
  // against 194 us), and a last front that the peel ordered will mostly be followed by another.
  const bool one_ordering_launch = peel_orders && opt().tail_merged && L.m <= 3 && last_outcome != 2;
  if (stepped) {
    // distances of the rows of the last front (the mask rank == worst), the order by (rank, distance descending, index)
    // from three stable argsort steps, the gather: the fitness is read from its structure-of-arrays copy
    WideLayout WL;
    if (!make_wide_layout(n, m, &WL) || WL.total > L.wide_bytes) return kErrWorkspace;
    uint8_t* wb = w.base + L.wide;
    int* const wide_outcome = opt().launch_memory ? outcome_slot(n, m, may_allocate, s, 1) : nullptr;
    if (wide_direct_applies(n, wide_outcome)) {
      if (int e = wide_select_direct(WL, wb, w.at<float>(L.xs), kWideFloat32, 1, L.npad, w.at<int>(L.rank), w.at<float>(L.dist), 1,
                                     w.at<int>(L.order), s, wide_outcome))
        return e;
      g.outcome = nullptr;
      launch_gather(false);
      EVX_LAUNCH_CHECK();
      return 0;
    }
    if (int e = wide_distances(WL, wb, w.at<float>(L.xs), kWideFloat32, 1, L.npad, nullptr, 0, w.at<int>(L.rank), w.at<float>(L.dist), 1,
                               true, s, wide_outcome))
      return e;
    int* order_a = reinterpret_cast<int*>(wb + WL.order_a);
    int* order_b = reinterpret_cast<int*>(wb + WL.order_b);
    void* sort_ws = wb + WL.sort_ws;
    if (int e = evox_hip_stable_argsort_step(wb + WL.neg_lo, kKeyUint32, 1, n, nullptr, order_a, sort_ws, WL.sort_bytes, s)) return e;
    if (int e = evox_hip_stable_argsort_step(wb + WL.neg_hi, kKeyUint32, 1, n, order_a, order_b, sort_ws, WL.sort_bytes, s)) return e;
    if (int e = evox_hip_stable_argsort_step(w.at<int>(L.rank), kKeyInt32, 1, n, order_b, w.at<int>(L.order), sort_ws, WL.sort_bytes, s))
      return e;
    g.outcome = nullptr;
    launch_gather(false);
    EVX_LAUNCH_CHECK();
    return 0;
  }
  if (peel_always_orders) {
    launch_gather(true);
    EVX_LAUNCH_CHECK();
    return 0;
  }
  if (!one_ordering_launch) {
    if (int e = stage_crowd_sort(w, w.at<int>(L.perm), true, 2, s, peel_orders)) return e;
    if (int e = stage_crowd_finish(w, w.at<int>(L.perm), true, 2, s, peel_orders)) return e;
    if (peel_orders)
      launch_gather(true);
    else
      launch_gather(false);
    EVX_LAUNCH_CHECK();
    return 0;
  }
  // the peel kernel may have ordered the last front: one launch for what is left of the ordering (nothing, then) and
  // the gather
  const size_t lds = crowd_lds_bytes(L, 2);
  const bool mid = crowd_mid_sort(L);
  const bool wide = L.n <= kMidArgsortWideRows;
  const bool many = w.batch > 1;
  auto instance = [&](auto one, auto several) { return many ? reinterpret_cast<const void*>(several) : reinterpret_cast<const void*>(one); };
  const void* const kernel = !mid   ? instance(crowd_gather_kernel<kRadixThreads, 0, false>, crowd_gather_kernel<kRadixThreads, 0, true>)
                             : wide ? instance(crowd_gather_kernel<kMidArgsortThreads, 1, false>, crowd_gather_kernel<kMidArgsortThreads, 1, true>)
                                    : instance(crowd_gather_kernel<kMidArgsortThreads, 2, false>, crowd_gather_kernel<kMidArgsortThreads, 2, true>);
  if (int e = grant_dynamic_lds(kernel, lds)) return e;
  int grid = finish_grid(L, L.m);  // resident at once: at most two blocks of 256 threads per compute unit
  if (grid > device_cus() * 2) grid = device_cus() * 2;
  grid = shared_grid(grid, mid ? device_cus() : device_cus() * 2, w.batch);
  const CrowdArgs ca = crowd_args(w, w.at<int>(L.perm), false, 2);
  if (mid && wide && many)
    hipLaunchKernelGGL((crowd_gather_kernel<kMidArgsortThreads, 1, true>), dim3(grid, 1, w.batch), dim3(kMidArgsortThreads), lds, s, ca, g);
  else if (mid && wide)
    hipLaunchKernelGGL((crowd_gather_kernel<kMidArgsortThreads, 1, false>), dim3(grid), dim3(kMidArgsortThreads), lds, s, ca, g);
  else if (mid && many)
    hipLaunchKernelGGL((crowd_gather_kernel<kMidArgsortThreads, 2, true>), dim3(grid, 1, w.batch), dim3(kMidArgsortThreads), lds, s, ca, g);
  else if (mid)
    hipLaunchKernelGGL((crowd_gather_kernel<kMidArgsortThreads, 2, false>), dim3(grid), dim3(kMidArgsortThreads), lds, s, ca, g);
  else if (many)
    hipLaunchKernelGGL((crowd_gather_kernel<kRadixThreads, 0, true>), dim3(grid, 1, w.batch), dim3(kRadixThreads), lds, s, ca, g);
  else
    hipLaunchKernelGGL((crowd_gather_kernel<kRadixThreads, 0, false>), dim3(grid), dim3(kRadixThreads), lds, s, ca, g);
  EVX_LAUNCH_CHECK();
  return 0;
}

extern "C" {

int evox_hip_nd_environmental_selection(const void* x, int64_t x_row_bytes, int64_t x_row_stride_bytes, const float* f,
                                        int64_t n, int64_t m, int64_t sr, int64_t sc, int64_t topk, void* out_x,
                                        float* out_f, int32_t* out_rank, float* out_dist, int32_t* out_order, void* ws,
                                        size_t ws_bytes, void* stream) {
  if (f == nullptr) return kErrBadArg;
  return select_rows(x, x_row_bytes, x_row_stride_bytes, x, x_row_stride_bytes, one_part(f, n, sr, sc), n, m, topk, out_x,
                     out_f, out_rank, out_dist, out_order, ws, ws_bytes, (hipStream_t)stream, true);
}

int evox_hip_nd_environmental_selection_two_part(const void* x_a, int64_t x_a_row_stride_bytes, const void* x_b,
                                                 int64_t x_b_row_stride_bytes, int64_t x_row_bytes, const float* f_a,
                                                 int64_t n_a, int64_t f_a_stride_row, int64_t f_a_stride_col,
                                                 const float* f_b, int64_t n_b, int64_t f_b_stride_row,
                                                 int64_t f_b_stride_col, int64_t m, int64_t topk, void* out_x, float* out_f,
                                                 int32_t* out_rank, float* out_dist, int32_t* out_order, void* ws,
                                                 size_t ws_bytes, void* stream) {
  if (n_a < 0 || n_b < 0 || n_a > 0x7FFFFF00ll || n_b > 0x7FFFFF00ll) return kErrBadArg;
  // a part without rows may come with null pointers: it is never read, the other part stands in for it
  if (n_a == 0) {
    f_a = f_b;
    x_a = x_b;
  }
  if (n_b == 0) {
    f_b = f_a;
    x_b = x_a;
  }
  if (f_a == nullptr || f_b == nullptr) return kErrBadArg;
  const Fitness fit{f_a, f_a_stride_row, f_a_stride_col, n_a, f_b, f_b_stride_row, f_b_stride_col};
  return select_rows(x_a, x_row_bytes, x_a_row_stride_bytes, x_b, x_b_row_stride_bytes, fit, n_a + n_b, m, topk, out_x, out_f,
                     out_rank, out_dist, out_order, ws, ws_bytes, (hipStream_t)stream, true);
}

}  // extern "C"

// ---- Many populations of one shape (more rows than the one-workgroup kernel of batched.hpp takes): the stages of the
// pipeline run once for `share` populations at a time, population b in the workgroups with blockIdx.z == b on its own
// copy of the workspace.  The kernels whose workgroups wait for each other get 1 / share of the device each, so that
// all of them are resident together; that is possible where the peel keeps the matrix in LDS (up to 32 768 rows) and
// a population's matrix fits the LDS of its share of the compute units.  Reference: the batched loop of
// src/evox/operators/selection/non_dominate.py:107-125 (torch.vmap of the ranking, utils/op_register.py:26-51).
static int many_populations_share(const Layout& L, int64_t batch, int64_t stop_count) {
  if (const int two = many_two_share(L, batch, stop_count)) return two;  // every population a chain of workgroups (two.hpp)
  if (batch < 2 || opt().peel_stepped || !opt().peel_lds || L.n > 32768) return 0;
  if (!opt().mid_argsort && L.n > kRadixMinCandidates) return 0;  // (large last fronts would take the radix grid)
  int share = 4 * device_cus() / 9;  // at least eight sweeping workgroups and the lister per population, up to four on a compute unit
  if (share > batch) share = (int)batch;
  size_t lds = 0;
  while (share >= 2 && lds_peel_plan(L, &lds, share) == 0) --share;
  if (share < 2) return 0;
  // (two objectives where many_two_share does not apply -- the LDS sorter switched off: several populations are still
  // faster through the matrix kernels that they share than one after the other, unless few of them fit a launch)
  if (two_applies(L, stop_count) && share < 4 && L.n > 12288) return 0;
  const int64_t passes = (batch + share - 1) / share;
  return (int)((batch + passes - 1) / passes);  // even passes: 30 populations, 28 at a time at most -> 15 + 15
}

static size_t many_workspace_step(const Layout& L) { return align_up(L.total); }

extern "C" {

/* Workspace for evox_hip_many_*: one copy of the single-population workspace per population that shares a launch. */
size_t evox_hip_many_workspace_bytes(int64_t batch, int64_t n, int64_t m, int64_t stop_count) {
  Layout L;
  if (batch < 1 || !make_layout(n, m, &L)) return 0;
  const int share = many_populations_share(L, batch, stop_count);
  return many_workspace_step(L) * (size_t)(share > 1 ? share : 1);
}

int64_t evox_hip_many_populations_per_launch(int64_t batch, int64_t n, int64_t m, int64_t stop_count) {
  Layout L;
  if (batch < 1 || !make_layout(n, m, &L)) return 0;
  const int share = many_populations_share(L, batch, stop_count);
  return share > 1 ? share : 1;
}

int evox_hip_many_non_dominate_rank_until(const float* f, int64_t batch, int64_t n, int64_t m, int64_t stride_batch, int64_t sr,
                                          int64_t sc, int64_t stop_count, int32_t* rank_out, void* ws, size_t ws_bytes,
                                          void* stream) {
  Layout L;
  if (f == nullptr || rank_out == nullptr || batch < 1 || !make_layout(n, m, &L)) return kErrBadArg;
  const int share = many_populations_share(L, batch, stop_count);
  const size_t step = many_workspace_step(L);
  for (int64_t b0 = 0; b0 < batch;) {
    const int64_t left = batch - b0;
    const int count = share > 1 ? (int)(left < share ? left : share) : 1;
    const Fitness fit = one_part(f + b0 * stride_batch, n, sr, sc, stride_batch);
    if (int e = rank_rows(fit, n, m, stop_count, rank_out + b0 * n, ws, ws_bytes, (hipStream_t)stream, count, count > 1 ? (int64_t)step : 0))
      return e;
    b0 += count;
  }
  return 0;
}

int evox_hip_many_nd_environmental_selection(const void* x, int64_t x_row_bytes, int64_t x_row_stride_bytes,
                                             int64_t x_batch_stride_bytes, const float* f, int64_t batch, int64_t n, int64_t m,
                                             int64_t stride_batch, int64_t sr, int64_t sc, int64_t topk, void* out_x, float* out_f,
                                             int32_t* out_rank, float* out_dist, void* ws, size_t ws_bytes, void* stream) {
  Layout L;
  if (f == nullptr || batch < 1 || !make_layout(n, m, &L) || topk < 1 || topk > n) return kErrBadArg;
  if ((x == nullptr) != (out_x == nullptr) || (x != nullptr && (x_row_bytes < 0 || x_batch_stride_bytes < 0))) return kErrBadArg;
  const int share = many_populations_share(L, batch, topk);
  const size_t step = many_workspace_step(L);
  for (int64_t b0 = 0; b0 < batch;) {
    const int64_t left = batch - b0;
    const int count = share > 1 ? (int)(left < share ? left : share) : 1;
    const Fitness fit = one_part(f + b0 * stride_batch, n, sr, sc, stride_batch);
    const uint8_t* xb = x != nullptr ? static_cast<const uint8_t*>(x) + b0 * x_batch_stride_bytes : nullptr;
    uint8_t* oxb = out_x != nullptr ? static_cast<uint8_t*>(out_x) + b0 * topk * x_row_bytes : nullptr;
    if (int e = select_rows(xb, x_row_bytes, x_row_stride_bytes, xb, x_row_stride_bytes, fit, n, m, topk, oxb, out_f + b0 * topk * m,
                            out_rank + b0 * topk, out_dist + b0 * topk, nullptr, ws, ws_bytes, (hipStream_t)stream, true, count,
                            count > 1 ? (int64_t)step : 0, x_batch_stride_bytes, x_batch_stride_bytes))
      return e;
    b0 += count;
  }
  return 0;
}

}  // extern "C"

extern "C" {

int evox_hip_dense_rank_rows(const void* sorted, int kind, const int64_t* index, int64_t batch, int64_t n, int64_t m, float* out,
                             void* stream) {
  if (sorted == nullptr || index == nullptr || out == nullptr || (kind != kWideFloat64 && kind != kWideInt64)) return kErrBadArg;
  if (batch < 1 || n < 1 || m < 1 || n >= (1ll << 24) || batch * m > 0x7FFFFFFFll) return kErrBadArg;
  hipStream_t s = (hipStream_t)stream;
  if (kind == kWideFloat64)
    hipLaunchKernelGGL(dense_rank_kernel<double>, dim3((unsigned)(batch * m)), dim3(kDenseRankThreads), 0, s,
                       static_cast<const double*>(sorted), index, (int)n, (int)m, out);
  else
    hipLaunchKernelGGL(dense_rank_kernel<long long>, dim3((unsigned)(batch * m)), dim3(kDenseRankThreads), 0, s,
                       static_cast<const long long*>(sorted), index, (int)n, (int)m, out);
  EVX_LAUNCH_CHECK();
  return 0;
}

size_t evox_hip_wide_workspace_bytes(int64_t n, int64_t m) {
  WideLayout L;
  return make_wide_layout(n, m, &L) ? L.total : 0;
}

int evox_hip_crowding_distance_wide(const void* costs, int kind, int64_t n, int64_t m, int64_t sr, int64_t sc, const uint8_t* mask,
                                    int64_t mask_stride, void* dist_out, int out_kind, void* ws, size_t ws_bytes, void* stream) {
  WideLayout L;
  if (costs == nullptr || dist_out == nullptr || (kind != kWideFloat64 && kind != kWideInt64) || (out_kind != 0 && out_kind != 1))
    return kErrBadArg;
  if (!make_wide_layout(n, m, &L)) return kErrBadArg;
  if (ws == nullptr || ws_bytes < L.total || (reinterpret_cast<uintptr_t>(ws) & 255u) != 0) return kErrWorkspace;
  return wide_distances(L, static_cast<uint8_t*>(ws), costs, kind, sr, sc, mask, mask_stride, nullptr, dist_out, out_kind, false,
                        (hipStream_t)stream);
}

int evox_hip_nd_environmental_selection_wide(const void* x, int64_t x_row_bytes, int64_t x_row_stride_bytes, const void* f_rows,
                                             int64_t f_row_bytes, int64_t f_row_stride_bytes, const void* costs, int kind, int64_t n,
                                             int64_t m, int64_t sr, int64_t sc, const int32_t* rank, int64_t topk, void* out_x,
                                             void* out_f, int32_t* out_rank, void* out_dist, int out_kind, void* ws, size_t ws_bytes,
                                             void* stream) {
  WideLayout L;
  if (costs == nullptr || rank == nullptr || f_rows == nullptr || out_f == nullptr || out_rank == nullptr || out_dist == nullptr)
    return kErrBadArg;
  if ((kind != kWideFloat64 && kind != kWideInt64) || (out_kind != 0 && out_kind != 1)) return kErrBadArg;
  if ((x == nullptr) != (out_x == nullptr) || x_row_bytes < 0 || x_row_stride_bytes < 0 || f_row_bytes < 1 || f_row_stride_bytes < 0)
    return kErrBadArg;
  if (!make_wide_layout(n, m, &L) || topk < 1 || topk > n) return kErrBadArg;
  if (ws == nullptr || ws_bytes < L.total || (reinterpret_cast<uintptr_t>(ws) & 255u) != 0) return kErrWorkspace;
  hipStream_t s = (hipStream_t)stream;
  uint8_t* base = static_cast<uint8_t*>(ws);
  void* dist = base + L.dist;
  int* order_a = reinterpret_cast<int*>(base + L.order_a);
  int* order_b = reinterpret_cast<int*>(base + L.order_b);
  int* const outcome = opt().launch_memory ? outcome_slot(n, m, true, s, 1) : nullptr;
  if (wide_direct_applies(n, outcome)) {
    if (int e = wide_select_direct(L, base, costs, kind, sr, sc, rank, dist, out_kind, order_a, s, outcome)) return e;
  } else {
    if (int e = wide_distances(L, base, costs, kind, sr, sc, nullptr, 0, rank, dist, out_kind, true, s, outcome)) return e;
    // rows by rank, then by distance descending (NaN last), then by index: one stable step per key part, least
    // significant first (src/evox/operators/selection/non_dominate.py:253, src/evox/utils/jit_fix_operator.py:246-250)
    void* sort_ws = base + L.sort_ws;
    if (int e = evox_hip_stable_argsort_step(base + L.neg_lo, kKeyUint32, 1, n, nullptr, order_a, sort_ws, L.sort_bytes, s)) return e;
    if (int e = evox_hip_stable_argsort_step(base + L.neg_hi, kKeyUint32, 1, n, order_a, order_b, sort_ws, L.sort_bytes, s)) return e;
    if (int e = evox_hip_stable_argsort_step(rank, kKeyInt32, 1, n, order_b, order_a, sort_ws, L.sort_bytes, s)) return e;
  }
  const int64_t dist_bytes = out_kind == 0 ? 8 : 4;
  const WideGather gather = {x, x_row_bytes, x_row_stride_bytes, 0, f_rows, f_row_bytes, f_row_stride_bytes, 0, rank, dist, dist_bytes, 0,
                             out_x, out_f, out_rank, out_dist};
  return wide_gather(gather, order_a, 0, n, topk, 1, s);
}

int evox_hip_many_nd_environmental_selection_wide(const void* x, int64_t x_row_bytes, int64_t x_row_stride_bytes, int64_t x_batch_stride_bytes,
                                                  const void* f_rows, int64_t f_row_bytes, int64_t f_row_stride_bytes,
                                                  int64_t f_batch_stride_bytes, const void* costs, int kind, int64_t batch, int64_t n,
                                                  int64_t m, int64_t stride_batch, int64_t sr, int64_t sc, const int32_t* rank,
                                                  int64_t topk, void* out_x, void* out_f, int32_t* out_rank, void* out_dist,
                                                  int out_kind, void* ws, size_t ws_bytes, void* stream) {
  WideLayout L;
  if (batch < 1 || !make_wide_layout(n, m, &L) || topk < 1 || topk > n) return kErrBadArg;
  if ((kind != kWideFloat64 && kind != kWideInt64) || (out_kind != 0 && out_kind != 1)) return kErrBadArg;
  const int64_t step = (int64_t)align_up(L.total);
  const int64_t dist_bytes = out_kind == 0 ? 8 : 4;
  hipStream_t s = (hipStream_t)stream;
  int* const outcome = opt().launch_memory ? outcome_slot(n, m, true, s, 1) : nullptr;
  const int64_t x_out_step = topk * x_row_bytes, f_out_step = topk * f_row_bytes;
  const bool together = batch > 1 && wide_direct_applies(n, outcome) && (n <= kSmallArgsortRows || opt().mid_argsort) &&
                        ws_bytes >= (size_t)step * (size_t)batch && batch <= 65535;
  if (!together) {  // one population after the other, each through the single-population entry point
    for (int64_t b = 0; b < batch; ++b) {
      const int e = evox_hip_nd_environmental_selection_wide(
          x ? static_cast<const char*>(x) + b * x_batch_stride_bytes : nullptr, x_row_bytes, x_row_stride_bytes,
          static_cast<const char*>(f_rows) + b * f_batch_stride_bytes, f_row_bytes, f_row_stride_bytes,
          static_cast<const char*>(costs) + b * stride_batch * 8, kind, n, m, sr, sc, rank + b * n, topk,
          out_x ? static_cast<char*>(out_x) + b * x_out_step : nullptr, static_cast<char*>(out_f) + b * f_out_step, out_rank + b * topk,
          static_cast<char*>(out_dist) + b * topk * dist_bytes, out_kind, ws, ws_bytes, stream);
      if (e) return e;
    }
    return 0;
  }
  if (costs == nullptr || rank == nullptr || f_rows == nullptr || out_f == nullptr || out_rank == nullptr || out_dist == nullptr)
    return kErrBadArg;
  if ((x == nullptr) != (out_x == nullptr) || x_row_bytes < 0 || x_row_stride_bytes < 0 || f_row_bytes < 1 || f_row_stride_bytes < 0)
    return kErrBadArg;
  if (ws == nullptr || (reinterpret_cast<uintptr_t>(ws) & 255u) != 0) return kErrWorkspace;
  uint8_t* base = static_cast<uint8_t*>(ws);
  void* dist = base + L.dist;
  int* order = reinterpret_cast<int*>(base + L.order_a);
  if (int e = wide_select_direct(L, base, costs, kind, sr, sc, rank, dist, out_kind, order, s, outcome, (int)batch, step, stride_batch * 8))
    return e;
  const WideGather gather = {x, x_row_bytes, x_row_stride_bytes, x_batch_stride_bytes, f_rows, f_row_bytes, f_row_stride_bytes,
                             f_batch_stride_bytes, rank, dist, dist_bytes, step, out_x, out_f, out_rank, out_dist};
  return wide_gather(gather, order, step, n, topk, (int)batch, s);
}

}  // extern "C"

// Scratch memory of the entry point that allocates nothing: part of the device image, one copy per GPU.  In host
// code the array's name stands for the symbol, not for device memory: its address on the current GPU comes from
// hipGetSymbolAddress, looked up once per device and kept.
static __device__ __align__(256) unsigned char scratch[EVOX_HIP_STATIC_SCRATCH_BYTES];
static std::atomic<void*> g_scratch_ptr[64];

static int static_scratch(void** out) {
  int dev = 0;
  const hipError_t de = hipGetDevice(&dev);
  if (de != hipSuccess) return (int)de;
  if (dev < 0 || dev >= 64) return kErrBadArg;
  void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (p == nullptr) {
    const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return (int)e;
    if (p == nullptr || (reinterpret_cast<uintptr_t>(p) & 255u) != 0) return kErrWorkspace;
    g_scratch_ptr[dev].store(p, std::memory_order_release);  // (two first calls at once look up the same address)
  }
  *out = p;
  return 0;
}

extern "C" {

int evox_hip_nd_environmental_selection_static(const void* x, int64_t x_row_bytes, int64_t x_row_stride_bytes,
                                               const float* f, int64_t n, int64_t m, int64_t sr, int64_t sc, int64_t topk,
                                               void* out_x, float* out_f, int32_t* out_rank, float* out_dist,
                                               int32_t* out_order, void* stream) {
  if (f == nullptr) return kErrBadArg;
  const size_t need = evox_hip_workspace_bytes(n, m);
  if (need == 0) return kErrBadArg;
  if (need > (size_t)EVOX_HIP_STATIC_SCRATCH_BYTES) return kErrStaticLimit;
  void* ws = nullptr;
  if (int e = static_scratch(&ws)) return e;
  // every call clears the part of the buffer that must start from zero (stage_prepare), whatever the call before
  // left there
  return select_rows(x, x_row_bytes, x_row_stride_bytes, x, x_row_stride_bytes, one_part(f, n, sr, sc), n, m, topk, out_x,
                     out_f, out_rank, out_dist, out_order, ws, (size_t)EVOX_HIP_STATIC_SCRATCH_BYTES, (hipStream_t)stream, false);
}

int64_t evox_hip_batched_max_rows(int64_t m) { return batched_rows_limit(m); }

int evox_hip_batched_non_dominate_rank(const float* f, int64_t batch, int64_t n, int64_t m, int64_t stride_batch,
                                       int64_t stride_row, int64_t stride_col, int32_t* rank_out, void* stream) {
  if (f == nullptr || rank_out == nullptr || batch < 1 || n < 1 || n > batched_rows_limit(m)) return kErrBadArg;
  BatchedArgs a = {};
  a.f = f;
  a.f_stride_b = stride_batch;
  a.f_stride_row = stride_row;
  a.f_stride_col = stride_col;
  a.n = (int)n;
  a.m = (int)m;
  a.stop_count = (int)n;
  a.rank_all = rank_out;
  return launch_batched(a, batch, (hipStream_t)stream);
}

int evox_hip_batched_nd_environmental_selection(const void* x, int64_t x_row_bytes, int64_t x_row_stride_bytes,
                                                int64_t x_batch_stride_bytes, const float* f, int64_t batch, int64_t n,
                                                int64_t m, int64_t stride_batch, int64_t stride_row, int64_t stride_col,
                                                int64_t topk, void* out_x, float* out_f, int32_t* out_rank, float* out_dist,
                                                void* stream) {
  if (f == nullptr || out_f == nullptr || out_rank == nullptr || out_dist == nullptr) return kErrBadArg;
  if (batch < 1 || n < 1 || n > batched_rows_limit(m) || topk < 1 || topk > n) return kErrBadArg;
  if ((x == nullptr) != (out_x == nullptr) || (x != nullptr && (x_row_bytes < 0 || x_row_stride_bytes < 0))) return kErrBadArg;
  BatchedArgs a = {};
  a.f = f;
  a.f_stride_b = stride_batch;
  a.f_stride_row = stride_row;
  a.f_stride_col = stride_col;
  a.n = (int)n;
  a.m = (int)m;
  a.stop_count = (int)topk;
  a.x = static_cast<const uint8_t*>(x);
  a.x_stride_b = x_batch_stride_bytes;
  a.x_row_stride = x_row_stride_bytes;
  a.x_row_bytes = x_row_bytes;
  a.out_x = static_cast<uint8_t*>(out_x);
  a.out_f = out_f;
  a.out_rank = out_rank;
  a.out_dist = out_dist;
  a.x_unit = 1;
  if (x != nullptr) {
    const uintptr_t bits = reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(out_x) | (uintptr_t)x_row_bytes |
                           (uintptr_t)x_row_stride_bytes | (uintptr_t)x_batch_stride_bytes;
    a.x_unit = (bits % 16 == 0) ? 16 : (bits % 4 == 0) ? 4 : 1;
  }
  return launch_batched(a, batch, (hipStream_t)stream);
}

int evox_hip_small_nd_environmental_selection_two_part(const void* x_a, const void* x_b, int64_t x_row_bytes,
                                                       int64_t x_row_stride_bytes, const float* f_a, int64_t n_a,
                                                       const float* f_b, int64_t n_b, int64_t m, int64_t stride_row,
                                                       int64_t stride_col, int64_t topk, void* out_x, float* out_f,
                                                       int32_t* out_rank, float* out_dist, void* stream) {
  if (f_a == nullptr || f_b == nullptr || out_f == nullptr || out_rank == nullptr || out_dist == nullptr) return kErrBadArg;
  if (n_a < 1 || n_b < 1 || n_a + n_b > batched_rows_limit(m)) return kErrBadArg;
  const int64_t n = n_a + n_b;
  if (topk < 1 || topk > n) return kErrBadArg;
  if ((x_a == nullptr) != (out_x == nullptr) || (x_a == nullptr) != (x_b == nullptr)) return kErrBadArg;
  if (x_a != nullptr && (x_row_bytes < 0 || x_row_stride_bytes < 0)) return kErrBadArg;
  BatchedArgs a = {};
  a.f = f_a;
  a.f_stride_row = stride_row;
  a.f_stride_col = stride_col;
  a.n = (int)n;
  a.m = (int)m;
  a.stop_count = (int)topk;
  a.n_first = (int)n_a;
  // row i >= n_a of the population is row i - n_a of part b: f_a + i * stride_row + f_second
  a.f_second = (f_b - f_a) - n_a * stride_row;
  a.x = static_cast<const uint8_t*>(x_a);
  a.x_row_stride = x_row_stride_bytes;
  a.x_row_bytes = x_row_bytes;
  a.out_x = static_cast<uint8_t*>(out_x);
  a.out_f = out_f;
  a.out_rank = out_rank;
  a.out_dist = out_dist;
  a.x_unit = 1;
  if (x_a != nullptr) {
    a.x_second = (static_cast<const uint8_t*>(x_b) - static_cast<const uint8_t*>(x_a)) - n_a * x_row_stride_bytes;
    const uintptr_t bits = reinterpret_cast<uintptr_t>(x_a) | reinterpret_cast<uintptr_t>(x_b) | reinterpret_cast<uintptr_t>(out_x) |
                           (uintptr_t)x_row_bytes | (uintptr_t)x_row_stride_bytes;
    a.x_unit = (bits % 16 == 0) ? 16 : (bits % 4 == 0) ? 4 : 1;
  }
  return launch_batched(a, 1, (hipStream_t)stream);
}

int evox_hip_tournament_pick(const int64_t* parents, int64_t n_round, int64_t tournament_size, const float* fit,
                             int64_t n_candidates, int64_t n_keys, int64_t stride_row, int64_t stride_col, int64_t* out,
                             void* stream) {
  if (parents == nullptr || fit == nullptr || out == nullptr) return kErrBadArg;
  if (n_round < 0 || tournament_size < 1 || tournament_size > 0x7FFFFFFF || n_candidates < 1 || n_keys < 1 || n_keys > 0x7FFFFFFF)
    return kErrBadArg;
  if (n_round == 0) return 0;
  int64_t blocks = (n_round + 255) / 256;
  if (blocks > 65535) blocks = 65535;
  hipLaunchKernelGGL(tournament_pick_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, parents, n_round,
                     (int)tournament_size, fit, stride_row, stride_col, (int)n_keys, out);
  EVX_LAUNCH_CHECK();
  return 0;
}

int evox_hip_tournament_pick_keys(const int64_t* parents, int64_t n_round, int64_t tournament_size, int64_t n_candidates,
                                  int64_t n_keys, const void* const* keys, const int32_t* kinds, const int64_t* strides,
                                  int64_t* out, void* stream) {
  if (parents == nullptr || keys == nullptr || kinds == nullptr || strides == nullptr || out == nullptr) return kErrBadArg;
  if (n_round < 0 || tournament_size < 1 || tournament_size > 0x7FFFFFFF || n_candidates < 1 || n_keys < 1 || n_keys > 4)
    return kErrBadArg;
  TournamentKeys t = {};
  for (int k = 0; k < (int)n_keys; ++k) {
    if (keys[k] == nullptr || (kinds[k] != 0 && kinds[k] != 1)) return kErrBadArg;
    t.key[k] = keys[k];
    t.kind[k] = kinds[k];
    t.stride[k] = strides[k];
  }
  t.nkeys = (int)n_keys;
  if (n_round == 0) return 0;
  int64_t blocks = (n_round + 255) / 256;
  if (blocks > 65535) blocks = 65535;
  hipLaunchKernelGGL(tournament_pick_keys_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, parents, n_round,
                     (int)tournament_size, t, out);
  EVX_LAUNCH_CHECK();
  return 0;
}

size_t evox_hip_hv_workspace_bytes(int64_t n, int64_t n_sample) {
  if (n < 1 || n_sample < 1 || n > 0x7FFFFF00ll || n_sample > 0x7FFFFF00ll) return 0;
  const int point_chunk = hv_chunk_length(n, kHvPointChunk), sample_chunk = hv_chunk_length(n_sample, kHvChunk);
  const size_t point_chunks = (size_t)((n + point_chunk - 1) / point_chunk);
  const size_t sample_chunks = (size_t)((n_sample + sample_chunk - 1) / sample_chunk);
  return align_up(sizeof(float) * (size_t)n_sample) + align_up(sizeof(int32_t) * point_chunks * (size_t)n_sample) +
         align_up(sizeof(float) * sample_chunks * (size_t)n);
}

int evox_hip_hv_contributions(const float* fit_t, const float* samples_t, const float* alpha, int64_t n, int64_t m,
                              int64_t n_sample, float scale, float* out, void* ws, size_t ws_bytes, void* stream) {
  if (fit_t == nullptr || samples_t == nullptr || alpha == nullptr || out == nullptr || m < 1 || m > 65535) return kErrBadArg;
  const size_t need = evox_hip_hv_workspace_bytes(n, n_sample);
  if (need == 0) return kErrBadArg;
  if (ws == nullptr || ws_bytes < need || (reinterpret_cast<uintptr_t>(ws) & 255u) != 0) return kErrWorkspace;
  hipStream_t s = (hipStream_t)stream;
  const int point_chunk = hv_chunk_length(n, kHvPointChunk), sample_chunk = hv_chunk_length(n_sample, kHvChunk);
  const int point_chunks = (int)((n + point_chunk - 1) / point_chunk);
  const int sample_chunks = (int)((n_sample + sample_chunk - 1) / sample_chunk);
  uint8_t* base = static_cast<uint8_t*>(ws);
  float* weight = reinterpret_cast<float*>(base);
  int32_t* cover = reinterpret_cast<int32_t*>(base + align_up(sizeof(float) * (size_t)n_sample));
  float* partial = reinterpret_cast<float*>(reinterpret_cast<uint8_t*>(cover) +
                                            align_up(sizeof(int32_t) * (size_t)point_chunks * (size_t)n_sample));
  const unsigned sample_blocks = (unsigned)((n_sample + 255) / 256), point_blocks = (unsigned)((n + 255) / 256);
  hipLaunchKernelGGL(hv_cover_count_kernel, dim3(sample_blocks, (unsigned)point_chunks), dim3(256), 0, s, fit_t, samples_t, (int)n,
                     (int)m, (int)n_sample, point_chunk, cover);
  EVX_LAUNCH_CHECK();
  hipLaunchKernelGGL(hv_sample_weight_kernel, dim3(sample_blocks), dim3(256), 0, s, cover, alpha, point_chunks, (int)n_sample,
                     weight);
  EVX_LAUNCH_CHECK();
  hipLaunchKernelGGL(hv_point_partial_kernel, dim3(point_blocks, (unsigned)sample_chunks), dim3(256), 0, s, fit_t, samples_t, weight,
                     (int)n, (int)m, (int)n_sample, sample_chunk, partial);
  EVX_LAUNCH_CHECK();
  hipLaunchKernelGGL(hv_point_total_kernel, dim3(point_blocks), dim3(256), 0, s, partial, (int)n, sample_chunks, scale, out);
  EVX_LAUNCH_CHECK();
  return 0;
}

size_t evox_hip_hv_covered_workspace_bytes(int64_t n_sample) {
  if (n_sample < 1 || n_sample > 0x7FFFFF00ll) return 0;
  return align_up(sizeof(uint32_t) * (size_t)n_sample);
}

int evox_hip_hv_covered_count(const float* points_t, const float* samples_t, int64_t n, int64_t m, int64_t n_sample,
                              int64_t* out_count, void* ws, size_t ws_bytes, void* stream) {
  if (points_t == nullptr || samples_t == nullptr || out_count == nullptr || n < 1 || n > 0x7FFFFF00ll || m < 1 || m > 65535)
    return kErrBadArg;
  const size_t need = evox_hip_hv_covered_workspace_bytes(n_sample);
  if (need == 0) return kErrBadArg;
  if (ws == nullptr || ws_bytes < need || (reinterpret_cast<uintptr_t>(ws) & 255u) != 0) return kErrWorkspace;
  const int64_t point_chunks = (n + kHvCoverChunk - 1) / kHvCoverChunk;
  if (point_chunks > 65535) return kErrBadArg;
  hipStream_t s = (hipStream_t)stream;
  uint32_t* flag = static_cast<uint32_t*>(ws);
  hipLaunchKernelGGL(reset_state_kernel, dim3(64), dim3(256), 0, s, flag, n_sample);
  EVX_LAUNCH_CHECK();
  hipLaunchKernelGGL(reset_state_kernel, dim3(1), dim3(64), 0, s, reinterpret_cast<uint32_t*>(out_count), (int64_t)2);
  EVX_LAUNCH_CHECK();
  const unsigned sample_blocks = (unsigned)((n_sample + 255) / 256);
  hipLaunchKernelGGL(hv_covered_kernel, dim3(sample_blocks, (unsigned)point_chunks), dim3(256), 0, s, points_t, samples_t, (int)n,
                     (int)m, (int)n_sample, flag);
  EVX_LAUNCH_CHECK();
  hipLaunchKernelGGL(hv_covered_total_kernel, dim3(sample_blocks < 64u ? sample_blocks : 64u), dim3(256), 0, s, flag, (int)n_sample,
                     reinterpret_cast<unsigned long long*>(out_count));
  EVX_LAUNCH_CHECK();
  return 0;
}

int evox_hip_calibration_launch(int kind, int64_t blocks, int64_t iterations, float* scratch_out, void* stream) {
  if (scratch_out == nullptr || kind < 0 || kind > 3 || blocks < 1 || blocks > 65535 || iterations < 1 || iterations > 10000000)
    return kErrBadArg;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)blocks), block(256);
  if (kind == 0)
    hipLaunchKernelGGL(calibrate_kernel<0>, grid, block, 0, s, scratch_out, (int)iterations, 1.0f, 2.0f);
  else if (kind == 1)
    hipLaunchKernelGGL(calibrate_kernel<1>, grid, block, 0, s, scratch_out, (int)iterations, 1.0f, 2.0f);
  else if (kind == 2)
    hipLaunchKernelGGL(calibrate_kernel<2>, grid, block, 0, s, scratch_out, (int)iterations, 1.0f, 2.0f);
  else
    hipLaunchKernelGGL(calibrate_kernel<3>, grid, block, 0, s, scratch_out, (int)iterations, 1.0f, 2.0f);
  EVX_LAUNCH_CHECK();
  return 0;
}

int evox_hip_dominance_plan(int64_t n, int64_t m, int64_t* out2) {
  Layout L;
  if (out2 == nullptr || !make_layout(n, m, &L)) return kErrBadArg;
  out2[0] = prefix_dominance_applies(L) ? 0 : dominance_tile_words(L);
  out2[1] = prefix_dominance_applies(L);
  return 0;
}

int evox_hip_peel_plan(int64_t n, int64_t m, int64_t* out3) {
  Layout L;
  if (out3 == nullptr || !make_layout(n, m, &L)) return kErrBadArg;
  size_t lds = 0;
  const int sweepers = lds_peel_plan(L, &lds);
  out3[0] = sweepers != 0;
  out3[1] = sweepers;
  out3[2] = (int64_t)lds;
  return 0;
}

int evox_hip_read_status(const void* ws, void* stream, int32_t* host_out8) {
  if (host_out8 == nullptr) return kErrBadArg;
  if (ws == nullptr) {  // the library's own scratch memory on the current device (the entry point that takes no workspace)
    void* own = nullptr;
    if (int e = static_scratch(&own)) return e;
    ws = own;
  }
  // the control block is the first region of the workspace
  hipError_t e = hipMemcpyAsync(host_out8, ws, 8 * sizeof(int32_t), hipMemcpyDeviceToHost, (hipStream_t)stream);
  if (e != hipSuccess) return (int)e;
  e = hipStreamSynchronize((hipStream_t)stream);
  if (e != hipSuccess) return (int)e;
  return host_out8[0];
}

}  // extern "C"
