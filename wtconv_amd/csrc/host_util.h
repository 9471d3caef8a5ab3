// Host-side helpers shared by the translation units of libwtconv_hip.so: the thread-local
// error message, kernel launch (HIP, or the host emulation), and driver queries that are
// looked up once per kernel.  Pure host code.
#pragma once

#include <stdarg.h>
#include <stdio.h>

#include <functional>
#include <mutex>
#include <unordered_map>

#include "common.h"

namespace wt {

inline thread_local char g_err[512] = "";

inline int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

#ifdef WT_EMULATE
#define WT_LAUNCH(kernel, grid, block, lds_bytes, stream, ...) \
  ::emu::launch((grid), (block), (lds_bytes), [&]() { kernel(__VA_ARGS__); })
inline int check_launch(const char*) { return 0; }
template <typename F> inline int allow_lds(F, size_t) { return 0; }
#else
#define WT_LAUNCH(kernel, grid, block, lds_bytes, stream, ...) \
  hipLaunchKernelGGL(kernel, (grid), (block), (lds_bytes), (stream), __VA_ARGS__)
inline int check_launch(const char* what) {
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(WTCONV_E_LAUNCH, "%s: %s", what, hipGetErrorString(e));
  return 0;
}
// Per-kernel facts that cost a driver call (hundreds of nanoseconds to microseconds each) are
// looked up once per (device, kernel, launch shape) and kept for the life of the process.
struct KernelKey {
  int dev; const void* fn; int block; size_t lds;
  bool operator==(const KernelKey& o) const { return dev == o.dev && fn == o.fn && block == o.block && lds == o.lds; }
};
struct KernelKeyHash {
  size_t operator()(const KernelKey& k) const {
    return std::hash<const void*>()(k.fn) ^ (static_cast<size_t>(k.dev) * 0x9e3779b97f4a7c15ull) ^
           (k.lds * 31 + static_cast<size_t>(k.block));
  }
};
inline std::mutex g_kernel_cache_mutex;
inline std::unordered_map<KernelKey, int, KernelKeyHash> g_lds_allowed, g_resident;

inline int current_device() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) { (void)hipGetLastError(); dev = 0; }
  return dev;
}

// Workgroups above 64 KiB of dynamic LDS need the opt-in attribute (set once per kernel and size).
template <typename F> inline int allow_lds(F kernel, size_t bytes) {
  if (bytes <= 64 * 1024) return 0;
  const KernelKey key = {current_device(), reinterpret_cast<const void*>(kernel), 0, bytes};
  {
    std::lock_guard<std::mutex> lock(g_kernel_cache_mutex);
    if (g_lds_allowed.count(key)) return 0;
  }
  const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize,
                                           static_cast<int>(bytes));
  if (e != hipSuccess) return fail(WTCONV_E_LAUNCH, "hipFuncSetAttribute(%zu B LDS): %s", bytes, hipGetErrorString(e));
  std::lock_guard<std::mutex> lock(g_kernel_cache_mutex);
  g_lds_allowed[key] = 1;
  return 0;
}
#endif

// Compute units of the current device (cached per thread; 256 on MI355X).
inline int compute_units() {
#ifdef WT_EMULATE
  return 2;
#else
  static thread_local int cached_dev = -1, cached_cu = 0;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 256;
  if (dev != cached_dev) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cached_dev = dev;
    cached_cu = n;
  }
  return cached_cu;
#endif
}

// Workgroups of `kernel` that fit on one CU at once (registers, LDS, wave slots): the grid
// of a persistent kernel must not exceed CUs x this, or the surplus runs as a second round.
template <typename F>
inline int resident_per_cu(F kernel, int block, size_t lds_bytes) {
#ifdef WT_EMULATE
  (void)kernel; (void)block; (void)lds_bytes;
  return 1;
#else
  const KernelKey key = {current_device(), reinterpret_cast<const void*>(kernel), block, lds_bytes};
  {
    std::lock_guard<std::mutex> lock(g_kernel_cache_mutex);
    auto it = g_resident.find(key);
    if (it != g_resident.end()) return it->second;
  }
  int n = 0;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, reinterpret_cast<const void*>(kernel), block, lds_bytes) !=
          hipSuccess || n < 1) {
    (void)hipGetLastError();
    const int by_lds = lds_bytes ? static_cast<int>(kLdsLimitBytes / lds_bytes) : 8;
    const int by_waves = 32 / (block / 64 > 0 ? block / 64 : 1);
    n = by_lds < by_waves ? by_lds : by_waves;
    if (n < 1) n = 1;
  }
  std::lock_guard<std::mutex> lock(g_kernel_cache_mutex);
  g_resident[key] = n;
  return n;
#endif
}

inline ParamTable to_table(const wtconv_params* p, int L) {
  ParamTable t = {};
  t.base_weight = p->base_weight;
  t.base_bias = p->base_bias;
  t.base_scale = p->base_scale;
  for (int l = 0; l < L; ++l) { t.wt_weight[l] = p->wt_weight[l]; t.wt_scale[l] = p->wt_scale[l]; }
  return t;
}

// Batch chunking of the 2-D weight-gradient kernel; a chunk is a whole number of
// iterations of `pb` planes.  `resident` = workgroups the device holds at once.
inline void wgrad_chunks(int B, int C, int pb, int resident, int* bchunk, int* nchunk) {
  // Chunks per channel n: C*n workgroups run in ceil(C*n/resident) rounds.  Every workgroup
  // pays LDS zeroing, a cold first fetch and the final reduction once, so score = fill of
  // the rounds minus 9 % per round, and the best n wins (ties: the smaller).  The penalty is
  // fitted to measurements (us per launch): 192 channels of 28x28 run best as 5 chunks (2 rounds,
  // 154) rather than 8 (3 full rounds, 168) or 2 (1 round three-quarters full, 177); 384
  // channels of 14x14 as 4 (131; 1 chunk: 145); 768 channels of 7x7 as 2; 96 channels of 56x56 as 5.
  const int iters = (B + pb - 1) / pb;           // iterations available per channel
  int best_n = 1;
  double best = -1.0;
  for (int n = 1; n <= iters && n <= 64; ++n) {
    const int wgs = C * n;
    const int rounds = (wgs + resident - 1) / resident;
    const double score = static_cast<double>(wgs) / (static_cast<double>(rounds) * resident) - 0.09 * rounds;
    if (score > best + 1e-9) { best = score; best_n = n; }
  }
  int bc = (iters + best_n - 1) / best_n * pb;
  if (bc < 1) bc = 1;
  *bchunk = bc;
  *nchunk = (B + bc - 1) / bc;
}

}  // namespace wt
