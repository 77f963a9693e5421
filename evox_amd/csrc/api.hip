// C ABI of libevox_hip.so (declared in include/evox_hip.h): argument checks, workspace layout
// and kernel launches.  Nothing here allocates device memory or waits for the device, except
// evox_hip_read_status().
#include <string.h>

#include "../../include/evox_hip.h"
#include "common.hpp"
#include "crowd.hpp"
#include "dominance.hpp"
#include "peel.hpp"

namespace evx {

constexpr int kMaxGrid = 4096;  // slots of the grid barrier

struct Options {
  int peel_blocks_per_cu = 2;
  unsigned spin_limit = 4000000u;
  int dominance_tile_words = 16;
};
static Options g_opt;

struct Layout {
  int n, m, npad, nwords, kstride;
  int64_t wstride;
  // byte offsets
  size_t ctrl, fsize, fronts, zero_end, fstart, xs, key, count, rank, dist, perm, order, ukey, pos, scost, dkey, dom, total;
};

static size_t align_up(size_t v) { return (v + 255) / 256 * 256; }

static bool make_layout(int64_t n, int64_t m, Layout* L) {
  if (n < 1 || m < 1 || n > 0x7FFFFF00ll || m > 65535) return false;
  L->n = (int)n;
  L->m = (int)m;
  L->npad = (int)round_up(n, 128);
  L->nwords = L->npad / 64;
  L->wstride = round_up(L->nwords, 16);
  L->kstride = (int)round_up(n, 64);
  size_t o = 0;
  // --- cleared by prepare_kernel on every call: control block, front sizes, front bitmaps
  L->ctrl = o;   o = align_up(o + sizeof(Ctrl) + sizeof(unsigned) * kMaxGrid);
  L->fsize = o;  o = align_up(o + sizeof(int) * (size_t)(n + 2));
  L->fronts = o; o = align_up(o + sizeof(uint64_t) * 3 * (size_t)L->nwords);
  L->zero_end = o;
  L->fstart = o; o = align_up(o + sizeof(int) * (size_t)(n + 2));
  L->xs = o;     o = align_up(o + sizeof(float) * (size_t)m * L->npad);
  L->key = o;    o = align_up(o + sizeof(uint64_t) * (size_t)L->npad);
  L->count = o;  o = align_up(o + sizeof(int) * (size_t)n);
  L->rank = o;   o = align_up(o + sizeof(int) * (size_t)n);
  L->dist = o;   o = align_up(o + sizeof(float) * (size_t)n);
  L->perm = o;   o = align_up(o + sizeof(int) * (size_t)n);
  L->order = o;  o = align_up(o + sizeof(int) * (size_t)n);
  L->ukey = o;   o = align_up(o + sizeof(uint32_t) * (size_t)m * L->kstride);
  L->pos = o;    o = align_up(o + sizeof(int) * (size_t)m * L->kstride);
  L->scost = o;  o = align_up(o + sizeof(float) * (size_t)m * L->kstride);
  L->dkey = o;   o = align_up(o + sizeof(uint32_t) * (size_t)L->kstride);
  L->dom = o;    o = align_up(o + sizeof(uint64_t) * (size_t)n * (size_t)L->wstride);
  L->total = o;
  return true;
}

struct Ws {
  Layout L;
  uint8_t* base;
  template <class T>
  T* at(size_t off) const {
    return reinterpret_cast<T*>(base + off);
  }
  Ctrl* ctrl() const { return at<Ctrl>(L.ctrl); }
};

static int open_ws(int64_t n, int64_t m, void* ws, size_t bytes, Ws* out) {
  if (!make_layout(n, m, &out->L)) return kErrBadArg;
  if (ws == nullptr || bytes < out->L.total || (reinterpret_cast<uintptr_t>(ws) & 255u) != 0) return kErrWorkspace;
  out->base = static_cast<uint8_t*>(ws);
  return 0;
}

static int device_cus() {
  static int cached[64] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (cached[dev] == 0) {
    int v = 0;
    if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0) v = 256;
    cached[dev] = v;
  }
  return cached[dev];
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
  dim3 grid((L.npad + 255) / 256, (L.nwords + IW - 1) / IW);
  if (variant == kDomTwoCompares)
    hipLaunchKernelGGL((dominance_kernel<M, IW, kDomTwoCompares>), grid, dim3(256), 0, s, w.at<float>(L.xs),
                       w.at<uint64_t>(L.key), w.at<uint64_t>(L.dom), L.n, L.npad, L.wstride, L.nwords);
  else
    hipLaunchKernelGGL((dominance_kernel<M, IW, kDomKey64>), grid, dim3(256), 0, s, w.at<float>(L.xs),
                       w.at<uint64_t>(L.key), w.at<uint64_t>(L.dom), L.n, L.npad, L.wstride, L.nwords);
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
      dim3 grid((L.npad + 255) / 256, (L.nwords + IW - 1) / IW);
      hipLaunchKernelGGL((dominance_any_m_kernel<IW>), grid, dim3(256), 0, s, w.at<float>(L.xs), w.at<uint64_t>(L.key),
                         w.at<uint64_t>(L.dom), L.n, L.npad, L.wstride, L.nwords, L.m);
    }
  }
}

static int stage_dominance(const Ws& w, const float* f, int64_t sr, int64_t sc, int variant, hipStream_t s) {
  const Layout& L = w.L;
  if (f == nullptr) return kErrBadArg;
  const int64_t zero_words = (int64_t)((L.zero_end - L.ctrl) / 4);
  int blocks = (int)((L.npad + 255) / 256);
  const int64_t zb = (zero_words + 255) / 256;
  if (zb > blocks) blocks = (int)(zb > 2048 ? 2048 : zb);
  hipLaunchKernelGGL(prepare_kernel, dim3(blocks), dim3(256), 0, s, f, sr, sc, L.n, L.m, L.npad, w.at<float>(L.xs),
                     w.at<uint64_t>(L.key), w.at<uint32_t>(L.ctrl), zero_words);
  EVX_LAUNCH_CHECK();
  // small populations get narrower tiles so that the grid still has many blocks
  int tile = g_opt.dominance_tile_words;
  if ((int64_t)((L.npad + 255) / 256) * ((L.nwords + 15) / 16) < 2 * device_cus()) tile = 4;
  if (tile >= 16)
    launch_dominance<16>(w, variant, s);
  else
    launch_dominance<4>(w, variant, s);
  EVX_LAUNCH_CHECK();
  return 0;
}

static int stage_count(const Ws& w, bool fill_dist, hipStream_t s) {
  const Layout& L = w.L;
  int blocks = (L.n + 3) / 4;
  const int cap = device_cus() * 8;
  if (blocks > cap) blocks = cap;
  hipLaunchKernelGGL(count_kernel, dim3(blocks), dim3(256), 0, s, w.at<uint64_t>(L.dom), L.wstride, L.nwords, L.n,
                     w.at<int>(L.count), w.at<int>(L.rank), w.at<uint64_t>(L.fronts), w.at<int>(L.fsize),
                     fill_dist ? w.at<float>(L.dist) : (float*)nullptr);
  EVX_LAUNCH_CHECK();
  return 0;
}

static int stage_peel(const Ws& w, int64_t stop_count, bool want_perm, hipStream_t s) {
  const Layout& L = w.L;
  if (stop_count < 1 || stop_count > L.n) return kErrBadArg;
  const size_t lds = sizeof(uint64_t) * (size_t)L.nwords;
  if (lds > 160 * 1024 - 4096) return kErrBadArg;
  if (lds > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(peel_kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return (int)e;
  }
  int per_cu = 0;
  hipError_t e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, peel_kernel, kPeelThreads, lds);
  if (e != hipSuccess) return (int)e;
  if (per_cu < 1) return kErrBadArg;
  if (per_cu > g_opt.peel_blocks_per_cu) per_cu = g_opt.peel_blocks_per_cu;
  // every block must be resident at once: the grid never exceeds what the device holds
  int blocks = device_cus() * per_cu;
  if (blocks > kMaxGrid) blocks = kMaxGrid;
  const int useful = 1 + (L.n + 3) / 4;  // block 0 + one wave per row
  if (blocks > useful) blocks = useful;
  hipLaunchKernelGGL(peel_kernel, dim3(blocks), dim3(kPeelThreads), lds, s, w.at<uint64_t>(L.dom), L.wstride, L.nwords,
                     L.n, w.at<int>(L.count), w.at<int>(L.rank), w.at<uint64_t>(L.fronts), w.at<int>(L.fsize),
                     want_perm ? w.at<int>(L.perm) : (int*)nullptr, w.at<int>(L.fstart), w.ctrl(), (int)stop_count,
                     g_opt.spin_limit);
  EVX_LAUNCH_CHECK();
  return 0;
}

// Crowding distance of the candidates list[ctrl.worst_start ... + ctrl.nv); dkey filled when the
// final ordering follows.
static int stage_crowding(const Ws& w, const int* list, bool want_dkey, hipStream_t s) {
  const Layout& L = w.L;
  int qblocks = (L.kstride + 255) / 256;
  if (qblocks > 4096) qblocks = 4096;
  hipLaunchKernelGGL(crowd_keys_kernel, dim3(qblocks, L.m), dim3(256), 0, s, w.at<float>(L.xs), L.npad, list, w.ctrl(),
                     w.at<uint32_t>(L.ukey), L.kstride);
  EVX_LAUNCH_CHECK();
  hipLaunchKernelGGL(crowd_rank_kernel, dim3(qblocks, L.m), dim3(256), 0, s, w.at<float>(L.xs), L.npad, list, w.ctrl(),
                     w.at<uint32_t>(L.ukey), L.kstride, w.at<int>(L.pos), w.at<float>(L.scost));
  EVX_LAUNCH_CHECK();
  hipLaunchKernelGGL(crowd_dist_kernel, dim3(qblocks), dim3(256), 0, s, list, w.ctrl(), L.m, w.at<int>(L.pos),
                     w.at<float>(L.scost), L.kstride, w.at<float>(L.dist),
                     want_dkey ? w.at<uint32_t>(L.dkey) : (uint32_t*)nullptr);
  EVX_LAUNCH_CHECK();
  return 0;
}

static int stage_order(const Ws& w, hipStream_t s) {
  const Layout& L = w.L;
  int blocks = (L.n + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  hipLaunchKernelGGL(final_order_kernel, dim3(blocks), dim3(256), 0, s, w.at<int>(L.perm), w.ctrl(), w.at<uint32_t>(L.dkey),
                     w.at<int>(L.order));
  EVX_LAUNCH_CHECK();
  return 0;
}

static int copy_async(void* dst, const void* src, size_t bytes, hipStream_t s) {
  return (int)hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, s);
}

}  // namespace evx

using namespace evx;

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
  return 0;
}

int evox_hip_set_option(const char* name, int64_t value) {
  if (name == nullptr) return kErrBadArg;
  if (!strcmp(name, "peel_blocks_per_cu") && value >= 1 && value <= 16) {
    g_opt.peel_blocks_per_cu = (int)value;
  } else if (!strcmp(name, "spin_limit") && value >= 1 && value <= 0x7FFFFFFFll) {
    g_opt.spin_limit = (unsigned)value;
  } else if (!strcmp(name, "dominance_tile_words") && (value == 4 || value == 16)) {
    g_opt.dominance_tile_words = (int)value;
  } else {
    return kErrBadArg;
  }
  return 0;
}

int evox_hip_stage_dominance(const float* f, int64_t n, int64_t m, int64_t sr, int64_t sc, int variant, void* ws,
                             size_t ws_bytes, void* stream) {
  Ws w;
  if (int e = open_ws(n, m, ws, ws_bytes, &w)) return e;
  return stage_dominance(w, f, sr, sc, variant, (hipStream_t)stream);
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
  if (int e = stage_peel(w, stop_count, true, (hipStream_t)stream)) return e;
  if (rank_out) return copy_async(rank_out, w.at<int>(w.L.rank), sizeof(int) * (size_t)n, (hipStream_t)stream);
  return 0;
}

int evox_hip_stage_crowding(int64_t n, int64_t m, void* ws, size_t ws_bytes, void* stream) {
  Ws w;
  if (int e = open_ws(n, m, ws, ws_bytes, &w)) return e;
  return stage_crowding(w, w.at<int>(w.L.perm), true, (hipStream_t)stream);
}

int evox_hip_stage_order(int64_t n, int64_t m, void* ws, size_t ws_bytes, void* stream) {
  Ws w;
  if (int e = open_ws(n, m, ws, ws_bytes, &w)) return e;
  return stage_order(w, (hipStream_t)stream);
}

int evox_hip_non_dominate_rank(const float* f, int64_t n, int64_t m, int64_t sr, int64_t sc, int32_t* rank_out, void* ws,
                               size_t ws_bytes, void* stream) {
  Ws w;
  if (rank_out == nullptr) return kErrBadArg;
  if (int e = open_ws(n, m, ws, ws_bytes, &w)) return e;
  hipStream_t s = (hipStream_t)stream;
  if (int e = stage_dominance(w, f, sr, sc, kDomKey64, s)) return e;
  if (int e = stage_count(w, false, s)) return e;
  if (int e = stage_peel(w, n, false, s)) return e;
  return copy_async(rank_out, w.at<int>(w.L.rank), sizeof(int) * (size_t)n, s);
}

int evox_hip_crowding_distance(const float* costs, int64_t n, int64_t m, int64_t sr, int64_t sc, const uint8_t* mask,
                               int64_t mask_stride, float* dist_out, void* ws, size_t ws_bytes, void* stream) {
  Ws w;
  if (costs == nullptr || dist_out == nullptr) return kErrBadArg;
  if (int e = open_ws(n, m, ws, ws_bytes, &w)) return e;
  const Layout& L = w.L;
  hipStream_t s = (hipStream_t)stream;
  const int64_t zero_words = (int64_t)((L.zero_end - L.ctrl) / 4);
  hipLaunchKernelGGL(prepare_kernel, dim3((L.npad + 255) / 256), dim3(256), 0, s, costs, sr, sc, L.n, L.m, L.npad,
                     w.at<float>(L.xs), w.at<uint64_t>(L.key), w.at<uint32_t>(L.ctrl), zero_words);
  EVX_LAUNCH_CHECK();
  hipLaunchKernelGGL(compact_mask_kernel, dim3(1), dim3(1024), 0, s, mask, mask_stride, L.n, w.at<int>(L.perm),
                     w.at<float>(L.dist), w.ctrl());
  EVX_LAUNCH_CHECK();
  if (int e = stage_crowding(w, w.at<int>(L.perm), false, s)) return e;
  return copy_async(dist_out, w.at<float>(L.dist), sizeof(float) * (size_t)n, s);
}

int evox_hip_nd_environmental_selection(const void* x, int64_t x_row_bytes, int64_t x_row_stride_bytes, const float* f,
                                        int64_t n, int64_t m, int64_t sr, int64_t sc, int64_t topk, void* out_x,
                                        float* out_f, int32_t* out_rank, float* out_dist, int32_t* out_order, void* ws,
                                        size_t ws_bytes, void* stream) {
  Ws w;
  if (out_f == nullptr || out_rank == nullptr || out_dist == nullptr) return kErrBadArg;
  if ((x == nullptr) != (out_x == nullptr) || (x != nullptr && (x_row_bytes < 0 || x_row_stride_bytes < 0))) return kErrBadArg;
  if (topk < 1 || topk > n) return kErrBadArg;
  if (int e = open_ws(n, m, ws, ws_bytes, &w)) return e;
  const Layout& L = w.L;
  hipStream_t s = (hipStream_t)stream;
  if (int e = stage_dominance(w, f, sr, sc, kDomKey64, s)) return e;
  if (int e = stage_count(w, true, s)) return e;
  if (int e = stage_peel(w, topk, true, s)) return e;
  if (int e = stage_crowding(w, w.at<int>(L.perm), true, s)) return e;
  if (int e = stage_order(w, s)) return e;
  int unit = 1;
  if (x != nullptr) {
    const uintptr_t bits = reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(out_x) | (uintptr_t)x_row_bytes |
                           (uintptr_t)x_row_stride_bytes;
    unit = (bits % 16 == 0) ? 16 : (bits % 4 == 0) ? 4 : 1;
  }
  int blocks = (int)((topk + 3) / 4);
  const int cap = device_cus() * 8;
  if (blocks > cap) blocks = cap;
  hipLaunchKernelGGL(gather_kernel, dim3(blocks), dim3(256), 0, s, w.at<int>(L.order), (int)topk,
                     static_cast<const uint8_t*>(x), x_row_stride_bytes, x_row_bytes, static_cast<uint8_t*>(out_x), unit, f,
                     sr, sc, L.m, out_f, w.at<int>(L.rank), out_rank, w.at<float>(L.dist), out_dist);
  EVX_LAUNCH_CHECK();
  if (out_order) return copy_async(out_order, w.at<int>(L.order), sizeof(int) * (size_t)topk, s);
  return 0;
}

int evox_hip_read_status(const void* ws, void* stream, int32_t* host_out8) {
  if (ws == nullptr || host_out8 == nullptr) return kErrBadArg;
  // the control block is the first region of the workspace
  hipError_t e = hipMemcpyAsync(host_out8, ws, 8 * sizeof(int32_t), hipMemcpyDeviceToHost, (hipStream_t)stream);
  if (e != hipSuccess) return (int)e;
  e = hipStreamSynchronize((hipStream_t)stream);
  if (e != hipSuccess) return (int)e;
  return host_out8[0];
}

}  // extern "C"
