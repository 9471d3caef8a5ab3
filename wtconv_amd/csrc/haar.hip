// Host side of the stand-alone Haar transforms (kernels_haar.h): argument checks and launches.  Allocates nothing,
// never synchronises.
#include <stdint.h>

#include "common.h"
#include "host_util.h"
#include "kernels_haar.h"

using namespace wt;

namespace {

int check_haar(const char* fn, const void* x, const void* out, long long units, int dtype) {
  if (x == nullptr || out == nullptr) return fail(WTCONV_E_ARG, "%s: null tensor pointer", fn);
  if (x == out) return fail(WTCONV_E_ARG, "%s: in-place use is not supported", fn);
  if (dtype != WTCONV_F32 && dtype != WTCONV_BF16 && dtype != WTCONV_F16) return fail(WTCONV_E_ARG, "%s: unknown dtype %d", fn, dtype);
  if (units <= 0) return fail(WTCONV_E_ARG, "%s: the number of planes / rows must be positive", fn);
  if (units > 65535LL * 65535LL) return fail(WTCONV_E_UNSUPPORTED, "%s: %lld planes / rows exceed the launch grid", fn, units);
  const size_t esz = dtype == WTCONV_F32 ? 4 : 2;
  if ((reinterpret_cast<uintptr_t>(x) % esz) || (reinterpret_cast<uintptr_t>(out) % esz))
    return fail(WTCONV_E_ARG, "%s: tensor pointer not aligned to its element size", fn);
  return 0;
}

dim3 unit_grid(unsigned gx, long long units) {
  const unsigned gy = units < 65535 ? static_cast<unsigned>(units) : 65535u;
  const unsigned gz = static_cast<unsigned>((units + gy - 1) / gy);
  return dim3(gx, gy, gz);
}

#define WT_HAAR_BY_DTYPE(dtype, CALL)                                          \
  do {                                                                         \
    if ((dtype) == WTCONV_F32) { using T_ = float; CALL; }                     \
    else if ((dtype) == WTCONV_BF16) { using T_ = bf16_t; CALL; }              \
    else { using T_ = f16_t; CALL; }                                           \
  } while (0)

}  // namespace

extern "C" int wtconv_haar2d(const void* x, void* out, long long planes, int H, int W, int dtype, int inverse,
                             void* stream_) {
  const char* fn = "wtconv_haar2d";
  if (int e = check_haar(fn, x, out, planes, dtype)) return e;
  if (H <= 0 || W <= 0 || H % 2 || W % 2)
    return fail(WTCONV_E_ARG, "%s: the plane must have even, positive extents (got %dx%d)", fn, H, W);
  if (static_cast<long long>(H) * W > (1LL << 30)) return fail(WTCONV_E_UNSUPPORTED, "%s: plane of %dx%d too large", fn, H, W);
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  const int h = H / 2, w = W / 2;
  const unsigned gx = static_cast<unsigned>((static_cast<long long>(h) * ((w + 1) / 2) + kHaarThreads - 1) / kHaarThreads);
  const dim3 grid = unit_grid(gx, planes);
  if (inverse)
    WT_HAAR_BY_DTYPE(dtype, WT_LAUNCH(haar2d_synthesis_kernel<T_>, grid, dim3(kHaarThreads), 0, stream,
                                      static_cast<const T_*>(x), static_cast<T_*>(out), h, w, planes));
  else
    WT_HAAR_BY_DTYPE(dtype, WT_LAUNCH(haar2d_analysis_kernel<T_>, grid, dim3(kHaarThreads), 0, stream,
                                      static_cast<const T_*>(x), static_cast<T_*>(out), h, w, planes));
  return check_launch(fn);
}

extern "C" int wtconv_haar1d(const void* x, void* out, long long rows, int N, int dtype, int inverse, void* stream_) {
  const char* fn = "wtconv_haar1d";
  if (int e = check_haar(fn, x, out, rows, dtype)) return e;
  if (N <= 0 || N % 2) return fail(WTCONV_E_ARG, "%s: the row length must be even and positive (got %d)", fn, N);
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  const int n = N / 2;
  const dim3 grid = unit_grid(static_cast<unsigned>((n + kHaarThreads - 1) / kHaarThreads), rows);
  WT_HAAR_BY_DTYPE(dtype, WT_LAUNCH(haar1d_kernel<T_>, grid, dim3(kHaarThreads), 0, stream, static_cast<const T_*>(x),
                                    static_cast<T_*>(out), n, rows, inverse));
  return check_launch(fn);
}
