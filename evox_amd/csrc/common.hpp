// Shared definitions for the gfx950 selection kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

// Hooks for development builds; they compile to nothing in the library.
#ifndef EVX_TRACE
#define EVX_TRACE(level, slot)
#endif

namespace evx {

constexpr int kWave = 64;

// Error codes returned through the C ABI (0 = ok, positive = hipError_t passed through).
constexpr int kErrBadArg = -1;
constexpr int kErrWorkspace = -2;
constexpr int kErrBarrierTimeout = -3;
constexpr int kErrStaticLimit = -4;

constexpr int kRankUnset = 0x7FFFFFFF;  // rank of a row that has not been peeled (yet)

__host__ __device__ inline int64_t round_up(int64_t v, int64_t q) { return (v + q - 1) / q * q; }

// Order-preserving map float -> uint32 with torch's sort conventions: -0.0 and +0.0 share a key,
// every NaN (either sign) maps to the largest key so that it sorts after +inf.
__device__ inline uint32_t ordered_key(float v) {
  uint32_t u = __float_as_uint(v);
  if (v != v) return 0xFFFFFFFFu;
  if (v == 0.0f) u = 0u;
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// Maximum, minimum and sum over the sixteen lanes of a group (lanes 16 g .. 16 g + 15), the same in every lane of
// the group: four rotations inside the DPP row (row_ror 8, 4, 2, 1), no trip through the LDS permute unit.
__device__ inline unsigned long long row16_rotate(unsigned long long v, int ctrl_index) {
  unsigned lo = (unsigned)v, hi = (unsigned)(v >> 32);
  switch (ctrl_index) {  // (the DPP control is an immediate)
    case 8:
      lo = __builtin_amdgcn_update_dpp(0, lo, 0x128, 0xf, 0xf, false);
      hi = __builtin_amdgcn_update_dpp(0, hi, 0x128, 0xf, 0xf, false);
      break;
    case 4:
      lo = __builtin_amdgcn_update_dpp(0, lo, 0x124, 0xf, 0xf, false);
      hi = __builtin_amdgcn_update_dpp(0, hi, 0x124, 0xf, 0xf, false);
      break;
    case 2:
      lo = __builtin_amdgcn_update_dpp(0, lo, 0x122, 0xf, 0xf, false);
      hi = __builtin_amdgcn_update_dpp(0, hi, 0x122, 0xf, 0xf, false);
      break;
    default:
      lo = __builtin_amdgcn_update_dpp(0, lo, 0x121, 0xf, 0xf, false);
      hi = __builtin_amdgcn_update_dpp(0, hi, 0x121, 0xf, 0xf, false);
      break;
  }
  return ((unsigned long long)hi << 32) | lo;
}
__device__ inline unsigned long long group16_max(unsigned long long v) {
#pragma unroll
  for (int r = 8; r >= 1; r >>= 1) {
    const unsigned long long o = row16_rotate(v, r);
    v = o > v ? o : v;
  }
  return v;
}
__device__ inline unsigned long long group16_min(unsigned long long v) {
#pragma unroll
  for (int r = 8; r >= 1; r >>= 1) {
    const unsigned long long o = row16_rotate(v, r);
    v = o < v ? o : v;
  }
  return v;
}
__device__ inline int group16_sum(int v) {
  v += __builtin_amdgcn_update_dpp(0, v, 0x128, 0xf, 0xf, false);
  v += __builtin_amdgcn_update_dpp(0, v, 0x124, 0xf, 0xf, false);
  v += __builtin_amdgcn_update_dpp(0, v, 0x122, 0xf, 0xf, false);
  v += __builtin_amdgcn_update_dpp(0, v, 0x121, 0xf, 0xf, false);
  return v;
}
// Several populations in one launch: population b is the workgroups with blockIdx.z == b, and every buffer of the
// library's workspace that a kernel is given for population 0 lies b * `step` bytes further on for population b (a
// launch for one population has blockIdx.z == 0 everywhere and passes a step of 0).  A kernel moves the pointers it
// was given once, at its start; a null pointer ("not wanted") stays null.
template <class P>
__device__ __forceinline__ void to_population(int64_t step_bytes, P& p) {
  if (p != nullptr) p = (P)((char*)p + (int64_t)blockIdx.z * step_bytes);
}
template <class P, class... More>
__device__ __forceinline__ void to_population(int64_t step_bytes, P& p, More&... more) {
  to_population(step_bytes, p);
  to_population(step_bytes, more...);
}

// Relaxed agent-scope accesses: one location at a time, coherent across the whole device, without
// the cache-wide write-back / invalidate that an agent-scope fence costs.  Everything that one
// block writes and another block reads during the kernel (front bitmaps, front sizes, barrier
// flags) is accessed only through these or through atomics.
template <class T>
__device__ inline T coherent_load(const T* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
template <class T>
__device__ inline void coherent_store(T* p, T v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// The bound of a device-side wait (the tunable "spin_limit").  A value up to kPollLimitMax counts failed polls (for
// tests that force a wait to give up: 1 ends it after the first failed poll, and every kernel still exits normally);
// a larger value is a time in ticks of the device's constant 100 MHz clock -- 10 ns; the default of 4 000 000 is
// 40 ms -- so that a wait ends after that time whatever else the device is doing, not after a number of polls whose
// duration depends on the load.  The clock is read on every 64th failed poll, the first reading starting the time.
constexpr unsigned kPollLimitMax = 65535u;
struct WaitBound {
  unsigned limit;
  unsigned long long t0;
  __device__ explicit WaitBound(unsigned l) : limit(l), t0(0ull) {}
  // after the failed poll number `spins` (counted from 0): must the wait end?
  __device__ bool expired(unsigned spins) {
    if (limit <= kPollLimitMax) return spins > limit;
    if ((spins & 63u) != 0u) return false;
    const unsigned long long now = (unsigned long long)wall_clock64();
    if (t0 == 0ull) {
      t0 = now | 1ull;
      return false;
    }
    return now - t0 > (unsigned long long)limit;
  }
};

// A wait on another workgroup that always ends: false when the bound `spin_limit` (WaitBound) ran out.
template <class Pred>
__device__ inline bool bounded_wait(Pred done, unsigned spin_limit) {
  unsigned spins = 0;
  WaitBound bound(spin_limit);
  while (!done()) {
    if (bound.expired(++spins)) return false;
    __builtin_amdgcn_s_sleep(1);
  }
  return true;
}

// Device control block shared by the peel / crowding / selection kernels of one call.
struct Ctrl {
  int err;          // 0, or kErrBarrierTimeout when a bounded grid-barrier wait ran out
  int nfronts;      // number of fronts peeled so far (ranks 0 .. nfronts-1 are final)
  int worst;        // rank of the front that contains the stop_count-th row
  int worst_start;  // rows ranked strictly better than `worst`
  int nv;           // size of front `worst`
  int need;         // rows to take from front `worst` (stop_count - worst_start)
  int passes;       // sweep passes executed
  int listed;       // front bitmaps 0 .. listed-1 have been listed and cleared; polled by the barrier master
  int radix_epoch;  // runs of a radix sort kernel so far: each takes a fresh range of barrier generations
  int tail_done;    // the peel kernel has also left the crowding distances and the order of the last front
  int reserved[6];  // [0], [1], [3]: arrival counters of the barriers inside the kernels that order the last front;
                    // [2]: that of the barriers inside the slot sort; [4]: the rounds that the last workgroup of
                    // the two-objective ranking went through (two.hpp); [5]: the level that the launch-per-front
                    // path has finished (stepped.hpp)
  // grid barrier: block 0 publishes (generation << 32 | rows found by all blocks) in `release` and in
  // kReleaseCopies copies of it, one per 128-byte line, so that the waiting blocks do not all poll one
  // address; all-ones means "give up" (a bounded wait ran out).  Every other block publishes
  // (generation << 32 | rows it found) in its own `arrive` slot.
  unsigned long long release;
  unsigned long long pad[15];
  unsigned long long release_copy[32 * 16];
  unsigned long long arrive[1];  // one slot per block (allocated to the grid size)
};
constexpr int kReleaseCopies = 32;
constexpr unsigned long long kReleaseGiveUp = ~0ull;

}  // namespace evx
