// Front peeling as one launch per front, for when the persistent peel kernels cannot be used.
//
// Reference semantics: the loop of src/evox/operators/selection/non_dominate.py:161-169 -- one short launch per front,
// which always makes progress whatever else the device is doing:
//   count -= (rows of the front just found that dominate the row); the rows whose count reaches zero form the next
//   front (:29-59).
// The persistent kernels of peel.hpp / peel_lds.hpp put all fronts into one launch whose workgroups wait for each
// other, which needs every workgroup resident at once: a device shared with another kernel, or one too small for the
// grid, cannot promise that, and the bounded waits then give up.  The kernel here waits for nobody: pass r reads the
// bitmap of front r - 1, which the pass before it has completed, lowers the counts of the unranked rows by the
// members of that front among their dominators (one coalesced sweep over the rows, the formulation of the reference),
// and collects the rows that reach zero as front r.  A few of its workgroups list front r - 1 in ascending original
// index.  The host launches passes in groups and looks at the control block between groups (the one place where this
// path waits for the stream).
#pragma once

#include "peel.hpp"

namespace evx {

constexpr int kStepThreads = 256;
constexpr int kStepListWords = kStepThreads;  // words of a front bitmap listed by one workgroup
constexpr int kStepDone = 5;                  // Ctrl.reserved[kStepDone]: level of the pass that found the ranking complete (0: none yet)

// Grid: `sweepers` sweeping workgroups, then ceil(nwords / kStepListWords) listing ones.  Dynamic LDS: nwords words.
// State: count (by slot; -1 once ranked, 0 for front 0), rank (by original index), the front bitmaps in rotation
// (front r in buffer r % kFrontBuffers, words kFrontStride apart), fsize, fstart, perm, the control block.
__global__ __launch_bounds__(kStepThreads) void step_pass_kernel(const uint64_t* __restrict__ dom, int64_t wstride, int nwords,
                                                                 int n, const int* __restrict__ orig_of, int* __restrict__ count,
                                                                 int* __restrict__ rank, uint64_t* __restrict__ fronts_slot,
                                                                 uint64_t* __restrict__ fronts_orig, int* __restrict__ fsize,
                                                                 int* __restrict__ fstart, int* __restrict__ perm,
                                                                 Ctrl* __restrict__ ctrl, int stop_count, int level, int sweepers) {
  extern __shared__ __attribute__((aligned(16))) uint64_t step_lds[];
  __shared__ int red[kStepThreads / 64];
  __shared__ int red_earlier[kStepThreads / 64];
  // (the flag holds the level of the pass that found the ranking complete: the workgroups of that very pass still
  // have its last front to list, those of later passes have nothing to do)
  const int done_at = ctrl->reserved[kStepDone];
  if (ctrl->err != 0 || (done_at != 0 && done_at != level)) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int prev = level - 1;
  const int before = prev == 0 ? 0 : fstart[prev];  // rows in the fronts before front `prev`
  const int size_prev = fsize[prev];
  const int total = before + size_prev;
  const bool done = size_prev <= 0 || total >= stop_count;
  const int64_t prev_buf = (int64_t)(prev % kFrontBuffers) * nwords * kFrontStride;
  if ((int)blockIdx.x >= sweepers) {
    // ---- listing of front `prev` (complete since the pass before): ascending original index into perm[before ...]
    if (perm == nullptr) return;
    const int first_word = ((int)blockIdx.x - sweepers) * kStepListWords;
    const uint64_t* bitmap = fronts_orig + prev_buf;
    int earlier = 0;  // members in the words before this workgroup's
    for (int w = tid; w < first_word; w += kStepThreads) earlier += __popcll(bitmap[(int64_t)w * kFrontStride]);
    earlier = wave_sum(earlier);
    const int w = first_word + tid;
    uint64_t bits = w < nwords ? bitmap[(int64_t)w * kFrontStride] : 0ull;
    const int mine = __popcll(bits);
    int incl = mine;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const int up = __shfl_up(incl, off);
      if (lane >= off) incl += up;
    }
    if (lane == 63) red[wave] = incl;
    if (lane == 0) red_earlier[wave] = earlier;
    __syncthreads();
    int pos = before + incl - mine;
    for (int v = 0; v < kStepThreads / 64; ++v) pos += red_earlier[v] + (v < wave ? red[v] : 0);
    while (bits) {
      perm[pos++] = w * 64 + __ffsll((unsigned long long)bits) - 1;
      bits &= bits - 1;
    }
    return;
  }
  if (blockIdx.x == 0 && tid == 0) {
    if (prev == 0) fstart[0] = 0;
    fstart[level] = total;
    if (done) {
      fstart[level] = total;
      ctrl->nfronts = level;
      ctrl->worst = prev;
      ctrl->worst_start = before;
      ctrl->nv = size_prev;
      ctrl->need = stop_count - before;
      ctrl->passes = prev;
    }
  }
  if (done) {
    if (blockIdx.x == 0 && tid == 0) ctrl->reserved[kStepDone] = level;
    return;
  }
  // ---- the sweep: front `prev` in slot space into LDS, then every unranked row against it
  const uint64_t* front = fronts_slot + prev_buf;
  for (int w = tid; w < ((nwords + 1) & ~1); w += kStepThreads) step_lds[w] = w < nwords ? front[(int64_t)w * kFrontStride] : 0ull;
  // the buffers of front level + 1 (they held front level + 1 - kFrontBuffers, listed passes ago) are cleared for the next pass
  {
    const int64_t next_buf = (int64_t)((level + 1) % kFrontBuffers) * nwords * kFrontStride;
    for (int w = (int)blockIdx.x * kStepThreads + tid; w < nwords; w += sweepers * kStepThreads) {
      fronts_slot[next_buf + (int64_t)w * kFrontStride] = 0ull;
      fronts_orig[next_buf + (int64_t)w * kFrontStride] = 0ull;
    }
  }
  __syncthreads();
  uint64_t* next_slot = fronts_slot + (int64_t)(level % kFrontBuffers) * nwords * kFrontStride;
  uint64_t* next_orig = fronts_orig + (int64_t)(level % kFrontBuffers) * nwords * kFrontStride;
  int found = 0;
  const int waves = sweepers * (kStepThreads / 64);
  for (int j = (int)blockIdx.x * (kStepThreads / 64) + wave; j < n; j += waves) {  // wave-uniform
    const int c = count[j];
    if (c <= 0) continue;  // ranked already
    const RowScan r = scan_row<true>(dom + (int64_t)j * wstride, row_words(j), step_lds);
    if (lane == 0) {
      const int left = c - r.total;
      count[j] = left == 0 ? -1 : left;
      if (left == 0) {
        const int o = orig_of[j];
        rank[o] = level;
        atomicOr(reinterpret_cast<unsigned long long*>(next_slot + (int64_t)(j >> 6) * kFrontStride), 1ull << (j & 63));
        atomicOr(reinterpret_cast<unsigned long long*>(next_orig + (int64_t)(o >> 6) * kFrontStride), 1ull << (o & 63));
        ++found;
      }
    }
  }
  if (lane == 0) red[wave] = found;
  __syncthreads();
  if (tid == 0) {
    int sum = 0;
    for (int v = 0; v < kStepThreads / 64; ++v) sum += red[v];
    if (sum) atomicAdd(&fsize[level], sum);
  }
}

}  // namespace evx
