// C ABI of libwtconv_hip.so (declared in include/wtconv_hip.h): argument checks, LDS
// planning and kernel launches.  Nothing here allocates, frees or synchronises.
#include <stdlib.h>
#include <string.h>

#include <mutex>

#include "common.h"
#include "host_util.h"
#include "mfma2d.h"
#include "kernels1d.h"
#include "kernels1d_row.h"
#include "kernels2d.h"
#include "kernels2d_stream.h"
#include "plan.h"

namespace wt {

// The element type of the activations as the template argument `T_` of a launcher call.
#define WT_BY_DTYPE(dtype, CALL)                                              \
  ((dtype) == WTCONV_F32 ? [&] { using T_ = float; return CALL; }()          \
   : (dtype) == WTCONV_BF16 ? [&] { using T_ = bf16_t; return CALL; }()      \
                            : [&] { using T_ = f16_t; return CALL; }())

// Threads of wgrad_finish_kernel: one per entry of a channel's record (taps of every filter + sumG) where that fits.
static inline int finish_threads(int nrec) { return nrec >= 1024 ? 1024 : (nrec + kWave - 1) / kWave * kWave; }

static inline bool known_dtype(int d) { return d == WTCONV_F32 || d == WTCONV_BF16 || d == WTCONV_F16; }

static int check_common(const char* fn, const wtconv_params* params, int B, int C, int K, int L,
                        int dtype, int pdtype) {
  if (B <= 0 || C <= 0) return fail(WTCONV_E_ARG, "%s: batch and channels must be positive (got %d, %d)", fn, B, C);
  if (K < 1 || K % 2 == 0) return fail(WTCONV_E_ARG, "%s: kernel_size must be odd and positive (got %d)", fn, K);
  if (K > wtconv_max_kernel_size())
    return fail(WTCONV_E_UNSUPPORTED, "%s: kernel_size %d exceeds the largest built kernel (%d)", fn, K,
                wtconv_max_kernel_size());
  if (L < 1 || L > kMaxLevels) return fail(WTCONV_E_ARG, "%s: wt_levels must be 1-%d (got %d)", fn, kMaxLevels, L);
  if (!known_dtype(dtype)) return fail(WTCONV_E_ARG, "%s: unknown dtype %d", fn, dtype);
  if (!known_dtype(pdtype)) return fail(WTCONV_E_ARG, "%s: unknown param dtype %d", fn, pdtype);
  if (params == nullptr || params->base_weight == nullptr || params->base_scale == nullptr)
    return fail(WTCONV_E_ARG, "%s: null parameter pointer", fn);
  for (int l = 0; l < L; ++l)
    if (params->wt_weight[l] == nullptr || params->wt_scale[l] == nullptr)
      return fail(WTCONV_E_ARG, "%s: null parameter pointer at level %d", fn, l);
  return 0;
}

// Workgroups of the weight-gradient kernel assumed resident when chunking the batch (2 per
// CU on 256 CUs).  A constant, so that workspace sizes do not depend on the device queried.
constexpr int kWgradResident = 512;

static size_t fold_floats(int C, int S, int L, int KK) { return static_cast<size_t>(C) * (1 + S * L) * KK + C; }

static int launch_fold(const wtconv_params* params, int pdtype, float* fw, float* fb, int C, int S, int L,
                       int KK, int flip, int use_bias, hipStream_t stream, unsigned* zero_words = nullptr,
                       int nzero = 0) {
  const int total = C * (1 + S * L) * KK;
  int blocks = (total + 255) / 256;
  if (blocks > 1024) blocks = 1024;
  WT_LAUNCH(fold_params_kernel, dim3(blocks), dim3(256), 0, stream, to_table(params, L), pdtype, fw, fb, C, S, L,
            KK, flip, use_bias, zero_words, zero_words != nullptr ? nzero : 0);
  return check_launch("fold_params_kernel");
}

// ---- 2-D dispatch over (dtype, K, level-1 strip width) -------------------------------
template <typename T, int K, int TJ1, int MODE, typename Geo = PlaneGeoRuntime>
static int run_plane2d_mode(const void* x, void* out, const float* fw, const float* fb, const Plan2D& pl,
                            hipStream_t stream) {
  auto kern = wt2d_plane_kernel<T, K, TJ1, kTJC, MODE, Geo>;
  const size_t lds = static_cast<size_t>(pl.lds_floats) * sizeof(float);
  if (int e = allow_lds(kern, lds)) return e;
  const int sg = 1 << pl.sg_shift;
  const int slots = pl.block / sg;
  const int nunits = sg < kWave ? (pl.C * pl.groups_per_channel + 3) / 4 : (pl.nplanes + slots - 1) / slots;
  int nwg = compute_units() * resident_per_cu(kern, pl.block, lds);
  if (nwg > nunits) nwg = nunits;
  WT_LAUNCH(kern, dim3(nwg), dim3(pl.block), lds, stream, static_cast<const T*>(x), static_cast<T*>(out), fw, fb, pl);
  return check_launch("wt2d_plane_kernel");
}

// Plane shapes of the WTConvNeXt stages with K = 5: geometry as a compile-time constant.  Returns 1 if the shape
// is not one of them (or the run-time plan differs, e.g. unaligned pointers), else the launch's result.
template <typename T>
static int run_plane2d_static(int K, int tj1, const void* x, void* out, const float* fw, const float* fb,
                              const Plan2D& pl, hipStream_t stream) {
  if (K != 5 || pl.H != pl.W) return 1;
#define WT_TRY(H_, L_)                                                                                  \
  if (pl.H == H_ && pl.L == L_) {                                                                       \
    using G = PlaneGeoStatic<H_, H_, 5, L_>;                                                            \
    constexpr Plan2D g = G::plan();                                                                     \
    if (tj1 == G::tj1() && same_plane_geometry(g, pl))                                                  \
      return run_plane2d_mode<T, 5, G::tj1(), G::mode(), G>(x, out, fw, fb, pl, stream);                \
    return 1;                                                                                           \
  }
  WT_TRY(56, 3) WT_TRY(28, 3) WT_TRY(14, 2) WT_TRY(7, 2)
#undef WT_TRY
  return 1;
}

template <typename T, int K, int TJ1>
static int run_plane2d(const void* x, void* out, const float* fw, const float* fb, const Plan2D& pl,
                       hipStream_t stream) {
  if (pl.prefetch && pl.fuse >= 2) return run_plane2d_mode<T, K, TJ1, 3>(x, out, fw, fb, pl, stream);
  if (pl.prefetch) return run_plane2d_mode<T, K, TJ1, 0>(x, out, fw, fb, pl, stream);
  if (pl.vec_ok) return run_plane2d_mode<T, K, TJ1, 1>(x, out, fw, fb, pl, stream);
  return run_plane2d_mode<T, K, TJ1, 2>(x, out, fw, fb, pl, stream);
}

template <typename T, int K>
static int run_plane2d_tj(int tj1, const void* x, void* out, const float* fw, const float* fb, const Plan2D& pl,
                          hipStream_t stream) {
  switch (tj1) {
    case 1: return run_plane2d<T, K, 1>(x, out, fw, fb, pl, stream);
    case 2: return run_plane2d<T, K, 2>(x, out, fw, fb, pl, stream);
    default: return run_plane2d<T, K, 4>(x, out, fw, fb, pl, stream);
  }
}

template <typename T>
static int run_plane2d_k(int K, int tj1, const void* x, void* out, const float* fw, const float* fb,
                         const Plan2D& pl, hipStream_t stream) {
  switch (K) {
    case 1: return run_plane2d_tj<T, 1>(tj1, x, out, fw, fb, pl, stream);
    case 3: return run_plane2d_tj<T, 3>(tj1, x, out, fw, fb, pl, stream);
    case 5: return run_plane2d_tj<T, 5>(tj1, x, out, fw, fb, pl, stream);
    case 7: return run_plane2d_tj<T, 7>(tj1, x, out, fw, fb, pl, stream);
  }
  return fail(WTCONV_E_UNSUPPORTED, "kernel_size %d is not built", K);
}

template <typename T, int K, int L, typename Geo = PlaneGeoRuntime>
static int run_wgrad2d(const void* x, const void* g, float* partial, const Plan2D& pl, int B, int bchunk,
                       int nchunk, const FinishArgs& fin, hipStream_t stream) {
  auto kern = wt2d_wgrad_kernel<T, K, L, kTJW, Geo>;
  const size_t lds = static_cast<size_t>(pl.lds_floats) * sizeof(float);
  if (int e = allow_lds(kern, lds)) return e;
  WT_LAUNCH(kern, dim3(pl.C, nchunk), dim3(512), lds, stream, static_cast<const T*>(x), static_cast<const T*>(g),
            partial, pl, B, bchunk, fin);
  return check_launch("wt2d_wgrad_kernel");
}

// Plane shapes of the WTConvNeXt stages with K = 5 at their usual planes per iteration: geometry as a compile-time
// constant.  Returns 1 if the launch is not one of them, else the launch's result.
template <typename T>
static int run_wgrad2d_static(int K, int L, const void* x, const void* g, float* partial, const Plan2D& pl, int B,
                              int bchunk, int nchunk, const FinishArgs& fin, hipStream_t stream) {
  if (K != 5 || pl.H != pl.W) return 1;
#define WT_TRY(H_, L_)                                                                                   \
  if (pl.H == H_ && L == L_) {                                                                           \
    constexpr int PB = wgrad_planes_per_iter(128, H_, H_, 5, L_);                                        \
    using G = WgradGeoStatic<H_, H_, 5, L_, PB>;                                                         \
    constexpr Plan2D gp = G::plan();                                                                     \
    if (same_wgrad_geometry(gp, pl))                                                                     \
      return run_wgrad2d<T, 5, L_, G>(x, g, partial, pl, B, bchunk, nchunk, fin, stream);                     \
    return 1;                                                                                            \
  }
  WT_TRY(56, 3) WT_TRY(28, 3) WT_TRY(14, 2) WT_TRY(7, 2)
#undef WT_TRY
  return 1;
}

template <typename T, int K>
static int run_wgrad2d_l(int L, const void* x, const void* g, float* partial, const Plan2D& pl, int B,
                         int bchunk, int nchunk, const FinishArgs& fin, hipStream_t stream) {
  switch (L) {
    case 1: return run_wgrad2d<T, K, 1>(x, g, partial, pl, B, bchunk, nchunk, fin, stream);
    case 2: return run_wgrad2d<T, K, 2>(x, g, partial, pl, B, bchunk, nchunk, fin, stream);
    case 3: return run_wgrad2d<T, K, 3>(x, g, partial, pl, B, bchunk, nchunk, fin, stream);
    case 4: return run_wgrad2d<T, K, 4>(x, g, partial, pl, B, bchunk, nchunk, fin, stream);
    case 5: return run_wgrad2d<T, K, 5>(x, g, partial, pl, B, bchunk, nchunk, fin, stream);
  }
  return fail(WTCONV_E_ARG, "wt_levels %d", L);
}

template <typename T>
static int run_wgrad2d_k(int K, int L, const void* x, const void* g, float* partial, const Plan2D& pl, int B,
                         int bchunk, int nchunk, const FinishArgs& fin, hipStream_t stream) {
  switch (K) {
    case 1: return run_wgrad2d_l<T, 1>(L, x, g, partial, pl, B, bchunk, nchunk, fin, stream);
    case 3: return run_wgrad2d_l<T, 3>(L, x, g, partial, pl, B, bchunk, nchunk, fin, stream);
    case 5: return run_wgrad2d_l<T, 5>(L, x, g, partial, pl, B, bchunk, nchunk, fin, stream);
    case 7: return run_wgrad2d_l<T, 7>(L, x, g, partial, pl, B, bchunk, nchunk, fin, stream);
  }
  return fail(WTCONV_E_UNSUPPORTED, "kernel_size %d is not built", K);
}

// ---- planes that do not fit LDS: level-by-level kernels through an HBM pyramid ----------
static size_t lds_fit_limit() {
#ifdef WT_EMULATE   // host emulation only: send small planes through the level-by-level kernels
  if (const char* e = getenv("WT_EMU_LDS_LIMIT")) return static_cast<size_t>(atol(e));
#endif
  return kLdsLimitBytes;
}

static bool plane_fits_lds(int B, int C, int H, int W, int K, int L) {
  Plan2D pl = make_plan2d(B, C, H, W, K, L, false, 256, 4, nullptr, nullptr, nullptr);
  return static_cast<size_t>(pl.plane_lds_floats) * 4 <= lds_fit_limit();
}

static bool wgrad_fits_lds(int B, int C, int H, int W, int K, int L) {
  Plan2D pl = make_plan2d(B, C, H, W, K, L, true, 512, 4, nullptr, nullptr, nullptr, 1);
  return static_cast<size_t>(pl.plane_lds_floats) * 4 <= lds_fit_limit();
}

static size_t round_up64(size_t v) { return (v + 63) / 64 * 64; }
constexpr long long kMaxPlaneElems = 1LL << 28;

static Stream2D make_stream2d(int B, int C, int H, int W, int L) {
  Stream2D s = {};
  s.C = C; s.H = H; s.W = W; s.L = L;
  s.nplanes = B * C;
  s.h[0] = H; s.w[0] = W;
  size_t off = 0;
  for (int l = 1; l <= L; ++l) {
    s.h[l] = (s.h[l - 1] + 1) / 2;
    s.w[l] = (s.w[l - 1] + 1) / 2;
    s.aoff[l] = off;
    off += round_up64(static_cast<size_t>(s.nplanes) * 4 * s.h[l] * s.w[l]);
  }
  for (int l = 2; l <= L; ++l) {
    s.zoff[l] = off;
    off += round_up64(static_cast<size_t>(s.nplanes) * s.h[l - 1] * s.w[l - 1]);
  }
  s.floats = off;
  return s;
}

// Chunks of the streamed weight-gradient kernels: the (batch item, tile) units of a level are
// split over `nchunk` workgroups per filter, about 2048 workgroups for the base-conv launch
// (C filters) and four times that for the sub-band launches, never more chunks than the
// finest level has units (a constant rule: workspace sizes do not depend on the device).
static int stream_chunks(int B, int C, int H, int W) {
  const long units = static_cast<long>(B) * ((H + kStreamTile - 1) / kStreamTile) *
                     ((W + kStreamTileW - 1) / kStreamTileW);
  long want = (2048 + C - 1) / C;
  if (want > 64) want = 64;
  if (want > units) want = units;
  if (want < 1) want = 1;
  return static_cast<int>(want);
}

static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// `ll_only`: the level-1 detail bands are not stored (forward / input-gradient pass: its last
// synthesis level rebuilds them from the pixels; the weight-gradient pass needs them).
template <typename T>
static int stream_analysis_chain(const T* src, float* pyr, const Stream2D& sp, hipStream_t stream, bool ll_only) {
  const unsigned gy = sp.nplanes < 65535 ? sp.nplanes : 65535;
  for (int l = 1; l <= sp.L; ++l) {
    const int n = sp.h[l] * sp.w[l];
    const unsigned gx = static_cast<unsigned>((n + 255) / 256);
    if (l == 1 && ll_only) {
      WT_LAUNCH((stream_analysis_kernel<T, true>), dim3(gx, gy), dim3(256), 0, stream, src,
                static_cast<size_t>(sp.H) * sp.W, sp.H, sp.W, pyr + sp.aoff[1], sp.h[1], sp.w[1], sp.nplanes);
    } else if (l == 1) {
      WT_LAUNCH((stream_analysis_kernel<T, false>), dim3(gx, gy), dim3(256), 0, stream, src,
                static_cast<size_t>(sp.H) * sp.W, sp.H, sp.W, pyr + sp.aoff[1], sp.h[1], sp.w[1], sp.nplanes);
    } else {
      WT_LAUNCH((stream_analysis_kernel<float, false>), dim3(gx, gy), dim3(256), 0, stream,
                static_cast<const float*>(pyr + sp.aoff[l - 1]), static_cast<size_t>(4) * sp.h[l - 1] * sp.w[l - 1],
                sp.h[l - 1], sp.w[l - 1], pyr + sp.aoff[l], sp.h[l], sp.w[l], sp.nplanes);
    }
    if (int e = check_launch("stream_analysis_kernel")) return e;
  }
  return 0;
}

// `have_pyramid`: the pyramid of x is in `pyr` already (the whole backward pass shares the one of grad_out).
template <typename T, int K>
static int run_stream2d(const void* x_, void* out_, const float* fw, const float* fb, float* pyr, const Stream2D& sp,
                        hipStream_t stream, bool have_pyramid = false) {
  const T* x = static_cast<const T*>(x_);
  T* out = static_cast<T*>(out_);
  if (sp.L > 1 && !have_pyramid) {      // a single level is synthesised from the pixels alone
    if (int e = stream_analysis_chain<T>(x, pyr, sp, stream, true)) return e;
  }
  const unsigned gy = sp.nplanes < 65535 ? sp.nplanes : 65535;
  const unsigned gz = (sp.nplanes + gy - 1) / gy;
  const int NF = 1 + 4 * sp.L;
  for (int l = sp.L; l >= 1; --l) {
    const unsigned tiles = static_cast<unsigned>(((sp.h[l] + kStreamTile - 1) / kStreamTile) *
                                                 ((sp.w[l] + kStreamTileW - 1) / kStreamTileW));
    const float* zin = l < sp.L ? pyr + sp.zoff[l + 1] : nullptr;
    const bool io_ok = l > 1 || (aligned16(x) && aligned16(out));
    const int vec = (sp.w[l] % 4 == 0 && aligned16(pyr) ? 1 : 0) | (sp.w[l - 1] % 4 == 0 && io_ok ? 2 : 0);
    if (l > 1) {
      WT_LAUNCH((stream_synth_kernel<T, K, false>), dim3(tiles, gy, gz), dim3(256), 0, stream,
                static_cast<const float*>(pyr + sp.aoff[l]), sp.h[l], sp.w[l], zin, pyr + sp.zoff[l], sp.h[l - 1],
                sp.w[l - 1], static_cast<const T*>(nullptr), static_cast<T*>(nullptr), fw, fb, sp.C, NF,
                1 + 4 * (l - 1), sp.nplanes, vec);
    } else {
      WT_LAUNCH((stream_synth_kernel<T, K, true>), dim3(tiles, gy, gz), dim3(256), 0, stream,
                static_cast<const float*>(pyr + sp.aoff[1]), sp.h[1], sp.w[1], zin, static_cast<float*>(nullptr), sp.H,
                sp.W, x, out, fw, fb, sp.C, NF, 1, sp.nplanes, vec);
    }
    if (int e = check_launch("stream_synth_kernel")) return e;
  }
  return 0;
}

template <typename T>
static int run_stream2d_k(int K, const void* x, void* out, const float* fw, const float* fb, float* pyr,
                          const Stream2D& sp, hipStream_t stream, bool have_pyramid = false) {
  switch (K) {
    case 1: return run_stream2d<T, 1>(x, out, fw, fb, pyr, sp, stream, have_pyramid);
    case 3: return run_stream2d<T, 3>(x, out, fw, fb, pyr, sp, stream, have_pyramid);
    case 5: return run_stream2d<T, 5>(x, out, fw, fb, pyr, sp, stream, have_pyramid);
    case 7: return run_stream2d<T, 7>(x, out, fw, fb, pyr, sp, stream, have_pyramid);
  }
  return fail(WTCONV_E_UNSUPPORTED, "kernel_size %d is not built", K);
}

// `have_g_pyramid`: the pyramid of grad_out is in `pyr_g` already (left there by the input-gradient pass of the same call).
template <typename T, int K>
static int run_stream2d_wgrad(const void* x_, const void* g_, float* partial, float* pyr_x, float* pyr_g,
                              const Stream2D& sp, int B, int nchunk, hipStream_t stream, bool have_g_pyramid = false) {
  const T* x = static_cast<const T*>(x_);
  const T* g = static_cast<const T*>(g_);
  if (int e = stream_analysis_chain<T>(x, pyr_x, sp, stream, false)) return e;
  if (!have_g_pyramid)
    if (int e = stream_analysis_chain<T>(g, pyr_g, sp, stream, false)) return e;
  const int rec = (1 + 4 * sp.L) * K * K + 1;
  const bool pyr_ok = aligned16(pyr_x) && aligned16(pyr_g);
  // chunks of a launch: at least four (batch item, tile) units per workgroup where the level has them
  auto level_chunks = [&](int h, int w) {
    const long units = static_cast<long>(B) * ((h + kStreamTile - 1) / kStreamTile) *
                       ((w + kStreamTileW - 1) / kStreamTileW);
    const long nc = units / 4;
    return static_cast<unsigned>(nc < 1 ? 1 : (nc > nchunk ? nchunk : nc));
  };
  WT_LAUNCH((stream_corr_kernel<T, K>), dim3(sp.C, level_chunks(sp.H, sp.W)), dim3(256), 0, stream, x, g,
            static_cast<size_t>(sp.H) * sp.W, static_cast<size_t>(0), sp.H, sp.W, partial, rec, 0, 1, 1, B, sp.C,
            (sp.W % 4 == 0 && aligned16(x) && aligned16(g)) ? 1 : 0, nchunk);
  if (int e = check_launch("stream_corr_kernel")) return e;
  for (int l = 1; l <= sp.L; ++l) {
    const size_t n = static_cast<size_t>(sp.h[l]) * sp.w[l];
    WT_LAUNCH((stream_corr_kernel<float, K>), dim3(sp.C * 4, level_chunks(sp.h[l], sp.w[l])), dim3(256), 0, stream,
              static_cast<const float*>(pyr_x + sp.aoff[l]), static_cast<const float*>(pyr_g + sp.aoff[l]), 4 * n, n,
              sp.h[l], sp.w[l], partial, rec, 1 + 4 * (l - 1), 4, 0, B, sp.C,
              (sp.w[l] % 4 == 0 && pyr_ok) ? 1 : 0, nchunk);
    if (int e = check_launch("stream_corr_kernel")) return e;
  }
  return 0;
}

template <typename T>
static int run_stream2d_wgrad_k(int K, const void* x, const void* g, float* partial, float* pyr_x, float* pyr_g,
                                const Stream2D& sp, int B, int nchunk, hipStream_t stream, bool have_g_pyramid = false) {
  switch (K) {
    case 1: return run_stream2d_wgrad<T, 1>(x, g, partial, pyr_x, pyr_g, sp, B, nchunk, stream, have_g_pyramid);
    case 3: return run_stream2d_wgrad<T, 3>(x, g, partial, pyr_x, pyr_g, sp, B, nchunk, stream, have_g_pyramid);
    case 5: return run_stream2d_wgrad<T, 5>(x, g, partial, pyr_x, pyr_g, sp, B, nchunk, stream, have_g_pyramid);
    case 7: return run_stream2d_wgrad<T, 7>(x, g, partial, pyr_x, pyr_g, sp, B, nchunk, stream, have_g_pyramid);
  }
  return fail(WTCONV_E_UNSUPPORTED, "kernel_size %d is not built", K);
}

// `shared_pyr` (level-by-level path only): where to build the whole pyramid of x -- detail bands of level 1 included --
// for a later pass of the same call to reuse; the folded parameters then go to `shared_fw` instead of the workspace start.
// `tickets` (plane-resident paths only): C words this pass clears on its way, for the parameter-gradient pass that
// follows it on the stream; they must lie outside the folded parameters at the workspace start.
static int plane2d_pass(const char* fn, const void* x, void* out, const wtconv_params* params, int B, int C,
                        int H, int W, int K, int L, int dtype, int pdtype, void* ws, size_t ws_bytes,
                        void* stream_, int flip, float* shared_pyr = nullptr, float* shared_fw = nullptr,
                        unsigned* tickets = nullptr) {
  if (int e = check_common(fn, params, B, C, K, L, dtype, pdtype)) return e;
  if (H <= 0 || W <= 0) return fail(WTCONV_E_ARG, "%s: spatial size must be positive (got %dx%d)", fn, H, W);
  if (static_cast<long long>(H) * W > kMaxPlaneElems)   // 32-bit offsets inside a plane and its four stacked sub-bands
    return fail(WTCONV_E_UNSUPPORTED, "%s: a plane of %dx%d exceeds 2^28 elements", fn, H, W);
  if (x == nullptr || out == nullptr) return fail(WTCONV_E_ARG, "%s: null tensor pointer", fn);
  const size_t esz = dtype == WTCONV_F32 ? 4 : 2;
  if ((reinterpret_cast<uintptr_t>(x) % esz) || (reinterpret_cast<uintptr_t>(out) % esz))
    return fail(WTCONV_E_ARG, "%s: tensor pointer not aligned to its element size", fn);
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  const size_t need = wtconv2d_workspace_bytes(B, C, H, W, K, L, flip ? WTCONV_PASS_BACKWARD_INPUT : WTCONV_PASS_FORWARD);
  if (ws == nullptr || ws_bytes < need)
    return fail(WTCONV_E_WORKSPACE, "%s: workspace of %zu B needed, %zu given", fn, need, ws_bytes);
  if (static_cast<long long>(B) * C > 0x7fffffffLL / 4)
    return fail(WTCONV_E_UNSUPPORTED, "%s: batch*channels = %lld is too large", fn, static_cast<long long>(B) * C);
  if (mfma2d_query(B, C, H, W, K, L, dtype).ok)
    return mfma2d_pass(fn, x, out, params, B, C, H, W, K, L, dtype, pdtype, stream, flip, tickets, C);
  if (!plane_fits_lds(B, C, H, W, K, L)) {
    const Stream2D sp = make_stream2d(B, C, H, W, L);
    float* fw = shared_pyr != nullptr ? shared_fw : static_cast<float*>(ws);
    float* fb = fw + static_cast<size_t>(C) * (1 + 4 * L) * K * K;
    float* pyr = shared_pyr != nullptr ? shared_pyr : fw + round_up64(fold_floats(C, 4, L, K * K));
    if (int e = launch_fold(params, pdtype, fw, fb, C, 4, L, K * K, flip, flip ? 0 : 1, stream)) return e;
    if (shared_pyr != nullptr) {
      if (int e = WT_BY_DTYPE(dtype, stream_analysis_chain<T_>(static_cast<const T_*>(x), pyr, sp, stream, false))) return e;
    }
    return WT_BY_DTYPE(dtype, run_stream2d_k<T_>(K, x, out, fw, fb, pyr, sp, stream, shared_pyr != nullptr));
  }
  Plan2D pl = make_plan2d(B, C, H, W, K, L, false, 256, esz, x, out, nullptr);
  int tj1 = 4, sg_shift = 8;
  choose_plane_shape(pl.h[1], pl.w[1], static_cast<size_t>(pl.plane_lds_floats) * 4, &tj1, &sg_shift);
  // keep the slots of a workgroup within LDS: fewer, larger plane groups if needed
  while (sg_shift < 8 && static_cast<size_t>(pl.plane_lds_floats) * 4 * (256 >> sg_shift) > kLdsLimitBytes / 2) ++sg_shift;
  finish_plane_plan(&pl, sg_shift);
  if (static_cast<size_t>(pl.lds_floats) * 4 > kLdsLimitBytes)
    return fail(WTCONV_E_UNSUPPORTED,
                "%s: a %dx%d plane with %d levels needs %zu B of LDS (limit %d); plane too large for the "
                "plane-resident kernels", fn, H, W, L, static_cast<size_t>(pl.lds_floats) * 4, kLdsLimitBytes);
  float* fw = static_cast<float*>(ws);
  float* fb = fw + static_cast<size_t>(C) * (1 + 4 * L) * K * K;
  if (int e = launch_fold(params, pdtype, fw, fb, C, 4, L, K * K, flip, flip ? 0 : 1, stream, tickets, C)) return e;
  if (dtype != WTCONV_BF16) {     // (bf16 tensors of these shapes are on the matrix-core kernels)
    const int e = dtype == WTCONV_F32 ? run_plane2d_static<float>(K, tj1, x, out, fw, fb, pl, stream)
                                      : run_plane2d_static<f16_t>(K, tj1, x, out, fw, fb, pl, stream);
    if (e != 1) return e;
  }
  return WT_BY_DTYPE(dtype, run_plane2d_k<T_>(K, tj1, x, out, fw, fb, pl, stream));
}

// ---- 1-D dispatch -------------------------------------------------------------------
template <typename T, int K>
static int run_tile1d(const void* x, void* out, const float* fw, const float* fb, const Plan1D& pl, int B,
                      hipStream_t stream) {
  auto kern = wt1d_tile_kernel<T, K, kTJ1D>;
  const size_t lds = static_cast<size_t>(pl.lds_floats) * sizeof(float);
  if (int e = allow_lds(kern, lds)) return e;
  const long long nrows = static_cast<long long>(B) * pl.C;
  if (nrows > 0x7fffffffLL) return fail(WTCONV_E_UNSUPPORTED, "batch*channels = %lld is too large", nrows);
  const unsigned gy = nrows < 65535 ? static_cast<unsigned>(nrows) : 65535u;
  const unsigned gz = static_cast<unsigned>((nrows + gy - 1) / gy);
  if (gz > 65535u) return fail(WTCONV_E_UNSUPPORTED, "batch*channels = %lld is too large", nrows);
  WT_LAUNCH(kern, dim3(pl.ntiles, gy, gz), dim3(kBlock1D), lds, stream, static_cast<const T*>(x),
            static_cast<T*>(out), fw, fb, pl, static_cast<int>(nrows));
  return check_launch("wt1d_tile_kernel");
}

template <typename T>
static int run_tile1d_k(int K, const void* x, void* out, const float* fw, const float* fb, const Plan1D& pl,
                        int B, hipStream_t stream) {
  switch (K) {
    case 1: return run_tile1d<T, 1>(x, out, fw, fb, pl, B, stream);
    case 3: return run_tile1d<T, 3>(x, out, fw, fb, pl, B, stream);
    case 5: return run_tile1d<T, 5>(x, out, fw, fb, pl, B, stream);
    case 7: return run_tile1d<T, 7>(x, out, fw, fb, pl, B, stream);
  }
  return fail(WTCONV_E_UNSUPPORTED, "kernel_size %d is not built", K);
}

template <typename T, int K, int L>
static int run_wgrad1d(const void* x, const void* g, float* partial, const Plan1D& pl, int B, int per_chunk,
                       int nchunk, hipStream_t stream) {
  auto kern = wt1d_wgrad_kernel<T, K, L, kTJ1D>;
  const size_t lds = static_cast<size_t>(pl.lds_floats) * sizeof(float);
  if (int e = allow_lds(kern, lds)) return e;
  WT_LAUNCH(kern, dim3(pl.C, nchunk), dim3(kBlock1D), lds, stream, static_cast<const T*>(x),
            static_cast<const T*>(g), partial, pl, B, per_chunk);
  return check_launch("wt1d_wgrad_kernel");
}

template <typename T, int K>
static int run_wgrad1d_l(int L, const void* x, const void* g, float* partial, const Plan1D& pl, int B,
                         int per_chunk, int nchunk, hipStream_t stream) {
  switch (L) {
    case 1: return run_wgrad1d<T, K, 1>(x, g, partial, pl, B, per_chunk, nchunk, stream);
    case 2: return run_wgrad1d<T, K, 2>(x, g, partial, pl, B, per_chunk, nchunk, stream);
    case 3: return run_wgrad1d<T, K, 3>(x, g, partial, pl, B, per_chunk, nchunk, stream);
    case 4: return run_wgrad1d<T, K, 4>(x, g, partial, pl, B, per_chunk, nchunk, stream);
    case 5: return run_wgrad1d<T, K, 5>(x, g, partial, pl, B, per_chunk, nchunk, stream);
  }
  return fail(WTCONV_E_ARG, "wt_levels %d", L);
}

template <typename T>
static int run_wgrad1d_k(int K, int L, const void* x, const void* g, float* partial, const Plan1D& pl, int B,
                         int per_chunk, int nchunk, hipStream_t stream) {
  switch (K) {
    case 1: return run_wgrad1d_l<T, 1>(L, x, g, partial, pl, B, per_chunk, nchunk, stream);
    case 3: return run_wgrad1d_l<T, 3>(L, x, g, partial, pl, B, per_chunk, nchunk, stream);
    case 5: return run_wgrad1d_l<T, 5>(L, x, g, partial, pl, B, per_chunk, nchunk, stream);
    case 7: return run_wgrad1d_l<T, 7>(L, x, g, partial, pl, B, per_chunk, nchunk, stream);
  }
  return fail(WTCONV_E_UNSUPPORTED, "kernel_size %d is not built", K);
}

// ---- row-resident 1-D kernels ----------------------------------------------------------
// Rows of 16 to `max_lanes` lanes' worth of samples run on the register-resident kernels, with 16 samples per lane
// where the row fits the workgroup that way and 32 otherwise; shorter or longer rows and K = 1 use the tiled ones.
struct Row1DShape { int S, nl, block; };

static bool row1d_shape(int N, int K, int L, int max_lanes, Row1DShape* sh) {
  if (K < 3 || K > 7 || L < 1 || L > kMaxLevels || N <= 0) return false;
  for (int S : {16, 32}) {
    if (!row1d_built(K, L, S)) continue;
    const int n = (N + S - 1) / S;
    if (n < 16 || n > max_lanes) continue;
    sh->S = S; sh->nl = n; sh->block = (n + 63) / 64 * 64;
    return true;
  }
  return false;
}

static Row1D make_row1d(int C, int N, int nl, size_t esz, const void* p0, const void* p1) {
  Row1D r = {};
  r.C = C; r.N = N; r.nl = nl;
  auto aligned = [](const void* p) { return p == nullptr || (reinterpret_cast<uintptr_t>(p) & 15u) == 0; };
  r.vec_ok = (static_cast<size_t>(N) * esz % 16 == 0) && aligned(p0) && aligned(p1);
  return r;
}

// Batch chunks of a row-resident kernel: C * nchunk workgroups that all run at once (one round: a second, partly
// filled round costs as much as a full one), `per_cu` of them per CU on 256 CUs -- constants, so that workspace
// sizes do not depend on the device queried.
static void row1d_chunks(int B, int C, int per_cu, int* per_chunk, int* nchunk) {
  if (per_cu < 1) per_cu = 1;
  int want = 256 * per_cu / C;
  if (want < 1) want = 1;
  if (want > B) want = B;
  const int pc = (B + want - 1) / want;
  *per_chunk = pc;
  *nchunk = (B + pc - 1) / pc;
}

// Workgroups per CU the kernels with two slot regions (parameter gradients, fused backward) are planned for: what
// LDS allows, at most two waves per SIMD (they need up to 256 registers).
static int row1d_two_region_per_cu(int K, int L, const Row1DShape& sh) {
  const size_t lds = 2 * row1d_region(K, L, sh.S, sh.block) * sizeof(float);
  int per_cu = static_cast<int>(kLdsLimitBytes / lds);
  if (per_cu > 512 / sh.block) per_cu = 512 / sh.block;
  return per_cu < 1 ? 1 : per_cu;
}

template <typename T, int K, int L, int S>
static int run_row1d(const void* x, void* out, const wtconv_params* params, int pdtype, int flip, const Row1D& pl,
                     int B, int block, hipStream_t stream) {
  if constexpr (row1d_built(K, L, S)) {
    auto kern = wt1d_row_kernel<T, K, L, S>;
    const size_t lds = row1d_region(K, L, S, block) * sizeof(float);
    if (int e = allow_lds(kern, lds)) return e;
    int per_chunk, nchunk;
    row1d_chunks(B, pl.C, resident_per_cu(kern, block, lds), &per_chunk, &nchunk);   // (no workspace depends on this)
    if (nchunk > 65535) return fail(WTCONV_E_UNSUPPORTED, "too many batch chunks (%d)", nchunk);
    WT_LAUNCH(kern, dim3(pl.C, nchunk), dim3(block), lds, stream, static_cast<const T*>(x), static_cast<T*>(out),
              to_table(params, L), pdtype, flip, pl, B, per_chunk);
    return check_launch("wt1d_row_kernel");
  } else {
    return fail(WTCONV_E_UNSUPPORTED, "row-resident 1-D kernel not built for kernel_size %d, %d levels", K, L);
  }
}

// The fused backward kernel: grad_x, the chunks' partial sums and (by the last workgroup of each channel) the
// parameter gradients.  `tickets`: C words, cleared by a launch of their own right before.
template <typename T, int K, int L, int S>
static int run_row1d_bwd(const void* x, const void* g, void* gx, float* partial, unsigned* tickets,
                         const wtconv_params* params, int pdtype, const GradTable& gt, const Row1D& pl, int B,
                         int block, int per_chunk, int nchunk, hipStream_t stream) {
  if constexpr (row1d_bwd_built(K, L, S)) {
    auto kern = wt1d_row_bwd_kernel<T, K, L, S>;
    const size_t lds = 2 * row1d_region(K, L, S, block) * sizeof(float);
    if (int e = allow_lds(kern, lds)) return e;
    WT_LAUNCH(zero_tickets_kernel, dim3((pl.C + 255) / 256), dim3(256), 0, stream, tickets, pl.C);
    if (int e = check_launch("zero_tickets_kernel")) return e;
    WT_LAUNCH(kern, dim3(pl.C, nchunk), dim3(block), lds, stream, static_cast<const T*>(x),
              static_cast<const T*>(g), static_cast<T*>(gx), partial, tickets, to_table(params, L), pdtype, gt, pl, B,
              per_chunk, nchunk);
    return check_launch("wt1d_row_bwd_kernel");
  } else {
    return fail(WTCONV_E_UNSUPPORTED, "row-resident 1-D kernel not built for kernel_size %d, %d levels", K, L);
  }
}

template <typename T, int K, int L, int S>
static int run_row1d_wgrad(const void* x, const void* g, float* partial, const Row1D& pl, int B, int block,
                           int per_chunk, int nchunk, hipStream_t stream) {
  if constexpr (row1d_built(K, L, S)) {
    auto kern = wt1d_row_wgrad_kernel<T, K, L, S>;
    const size_t lds = 2 * row1d_region(K, L, S, block) * sizeof(float);
    if (int e = allow_lds(kern, lds)) return e;
    WT_LAUNCH(kern, dim3(pl.C, nchunk), dim3(block), lds, stream, static_cast<const T*>(x),
              static_cast<const T*>(g), partial, pl, B, per_chunk);
    return check_launch("wt1d_row_wgrad_kernel");
  } else {
    return fail(WTCONV_E_UNSUPPORTED, "row-resident 1-D kernel not built for kernel_size %d, %d levels", K, L);
  }
}

#define WT_ROW1D_SWITCH_S(T, K, L, CALL)                              \
  return S == 16 ? CALL(T, K, L, 16) : CALL(T, K, L, 32);
#define WT_ROW1D_SWITCH_L(T, K, CALL)                                 \
  switch (L) {                                                        \
    case 1: WT_ROW1D_SWITCH_S(T, K, 1, CALL)                          \
    case 2: WT_ROW1D_SWITCH_S(T, K, 2, CALL)                          \
    case 3: WT_ROW1D_SWITCH_S(T, K, 3, CALL)                          \
    case 4: WT_ROW1D_SWITCH_S(T, K, 4, CALL)                          \
    case 5: WT_ROW1D_SWITCH_S(T, K, 5, CALL)                          \
  }                                                                   \
  break;
#define WT_ROW1D_SWITCH(T, CALL)                                      \
  switch (K) {                                                        \
    case 3: WT_ROW1D_SWITCH_L(T, 3, CALL)                             \
    case 5: WT_ROW1D_SWITCH_L(T, 5, CALL)                             \
    case 7: WT_ROW1D_SWITCH_L(T, 7, CALL)                             \
  }

template <typename T>
static int run_row1d_kl(int K, int L, int S, const void* x, void* out, const wtconv_params* params, int pdtype,
                        int flip, const Row1D& pl, int B, int block, hipStream_t stream) {
#define WT_CALL(T_, K_, L_, S_) run_row1d<T_, K_, L_, S_>(x, out, params, pdtype, flip, pl, B, block, stream)
  WT_ROW1D_SWITCH(T, WT_CALL)
#undef WT_CALL
  return fail(WTCONV_E_UNSUPPORTED, "kernel_size %d / %d levels not built", K, L);
}

template <typename T>
static int run_row1d_bwd_kl(int K, int L, int S, const void* x, const void* g, void* gx, float* partial,
                            unsigned* tickets, const wtconv_params* params, int pdtype, const GradTable& gt,
                            const Row1D& pl, int B, int block, int per_chunk, int nchunk, hipStream_t stream) {
#define WT_CALL(T_, K_, L_, S_)                                                                                 \
  run_row1d_bwd<T_, K_, L_, S_>(x, g, gx, partial, tickets, params, pdtype, gt, pl, B, block, per_chunk, nchunk, \
                                stream)
  WT_ROW1D_SWITCH(T, WT_CALL)
#undef WT_CALL
  return fail(WTCONV_E_UNSUPPORTED, "kernel_size %d / %d levels not built", K, L);
}

template <typename T>
static int run_row1d_wgrad_kl(int K, int L, int S, const void* x, const void* g, float* partial, const Row1D& pl,
                              int B, int block, int per_chunk, int nchunk, hipStream_t stream) {
#define WT_CALL(T_, K_, L_, S_) \
  run_row1d_wgrad<T_, K_, L_, S_>(x, g, partial, pl, B, block, per_chunk, nchunk, stream)
  WT_ROW1D_SWITCH(T, WT_CALL)
#undef WT_CALL
  return fail(WTCONV_E_UNSUPPORTED, "kernel_size %d / %d levels not built", K, L);
}

static int tile1d_pass(const char* fn, const void* x, void* out, const wtconv_params* params, int B, int C,
                       int N, int K, int L, int dtype, int pdtype, void* ws, size_t ws_bytes, void* stream_,
                       int flip) {
  if (int e = check_common(fn, params, B, C, K, L, dtype, pdtype)) return e;
  if (N <= 0) return fail(WTCONV_E_ARG, "%s: length must be positive (got %d)", fn, N);
  if (x == nullptr || out == nullptr) return fail(WTCONV_E_ARG, "%s: null tensor pointer", fn);
  const size_t esz = dtype == WTCONV_F32 ? 4 : 2;
  if ((reinterpret_cast<uintptr_t>(x) % esz) || (reinterpret_cast<uintptr_t>(out) % esz))
    return fail(WTCONV_E_ARG, "%s: tensor pointer not aligned to its element size", fn);
  Row1DShape sh = {};
  const bool row_resident = row1d_shape(N, K, L, kRow1dMaxLanes, &sh);
  const Plan1D pl = make_plan1d(C, N, K, L, false, esz, x, out, nullptr);
  const size_t need = wtconv1d_workspace_bytes(B, C, N, K, L, flip ? WTCONV_PASS_BACKWARD_INPUT : WTCONV_PASS_FORWARD);
  if (ws == nullptr || ws_bytes < need)
    return fail(WTCONV_E_WORKSPACE, "%s: workspace of %zu B needed, %zu given", fn, need, ws_bytes);
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  if (row_resident) {      // (these kernels fold their channel's parameters themselves: no fold launch, no table)
    const Row1D rp = make_row1d(C, N, sh.nl, esz, x, out);
    return WT_BY_DTYPE(dtype, run_row1d_kl<T_>(K, L, sh.S, x, out, params, pdtype, flip, rp, B, sh.block, stream));
  }
  float* fw = static_cast<float*>(ws);
  float* fb = fw + static_cast<size_t>(C) * (1 + 2 * L) * K;
  if (int e = launch_fold(params, pdtype, fw, fb, C, 2, L, K, flip, flip ? 0 : 1, stream)) return e;
  return WT_BY_DTYPE(dtype, run_tile1d_k<T_>(K, x, out, fw, fb, pl, B, stream));
}

// ---- static scratch for callers that may not allocate ------------------------------------
// One array per GPU the library runs on, held until the process ends.  Host code never uses the
// array's name as an address: the device address is looked up once per device and cached.
constexpr size_t kStaticScratchBytes = 4u << 20;
constexpr int kMaxDevices = 64;
#ifndef WT_EMULATE
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
static std::mutex g_scratch_mutex;
static void* g_scratch_ptr[kMaxDevices];

static int static_scratch(const char* fn, void** ptr) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail(WTCONV_E_LAUNCH, "%s: hipGetDevice: %s", fn, hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices) return fail(WTCONV_E_UNSUPPORTED, "%s: device index %d", fn, dev);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || p == nullptr)
      return fail(WTCONV_E_LAUNCH, "%s: hipGetSymbolAddress(scratch): %s", fn, hipGetErrorString(e));
    g_scratch_ptr[dev] = p;
  }
  *ptr = g_scratch_ptr[dev];
  return 0;
}
#else
static unsigned char scratch[kStaticScratchBytes];
static int static_scratch(const char*, void** ptr) { *ptr = scratch; return 0; }
#endif

static int check_grad_table(const char* fn, const wtconv_params* params, const wtconv_param_grads* grads, int L) {
  if (grads == nullptr) return fail(WTCONV_E_ARG, "%s: null tensor pointer", fn);
  if (grads->base_weight == nullptr || grads->base_scale == nullptr ||
      (params->base_bias != nullptr && grads->base_bias == nullptr))
    return fail(WTCONV_E_ARG, "%s: null gradient pointer", fn);
  for (int l = 0; l < L; ++l)
    if (grads->wt_weight[l] == nullptr || grads->wt_scale[l] == nullptr)
      return fail(WTCONV_E_ARG, "%s: null gradient pointer at level %d", fn, l);
  return 0;
}

static GradTable to_grad_table(const wtconv_param_grads* grads, int L) {
  GradTable gt = {};
  gt.base_weight = grads->base_weight;
  gt.base_bias = grads->base_bias;
  gt.base_scale = grads->base_scale;
  for (int l = 0; l < L; ++l) { gt.wt_weight[l] = grads->wt_weight[l]; gt.wt_scale[l] = grads->wt_scale[l]; }
  return gt;
}

}  // namespace wt

using namespace wt;

extern "C" {

int wtconv_abi_version(void) { return WTCONV_ABI_VERSION; }

const char* wtconv_last_error(void) { return g_err; }

int wtconv_max_kernel_size(void) { return 7; }

size_t wtconv2d_workspace_bytes(int B, int C, int H, int W, int K, int levels, int pass) {
  if (pass == WTCONV_PASS_BACKWARD) {
    const size_t a = wtconv2d_workspace_bytes(B, C, H, W, K, levels, WTCONV_PASS_BACKWARD_INPUT);
    const size_t b = wtconv2d_workspace_bytes(B, C, H, W, K, levels, WTCONV_PASS_BACKWARD_PARAMS);
    return a > b ? a : b;
  }
  if (B <= 0 || C <= 0 || H <= 0 || W <= 0 || K <= 0 || levels <= 0 || levels > kMaxLevels) return 0;
  if (static_cast<long long>(H) * W > kMaxPlaneElems) return 0;
  size_t floats;
  if (pass == WTCONV_PASS_BACKWARD_PARAMS) {
    int bchunk, nchunk;
    // the dtype is not an argument here: room for the bf16 matrix-core kernel's partial sums as well
    const Mfma2dWgradQuery mq = mfma2d_wgrad_query(B, C, H, W, K, levels, WTCONV_BF16);
    const size_t mfloats = mq.ok ? mq.ws_bytes / sizeof(float) : 0;
    if (wgrad_fits_lds(B, C, H, W, K, levels)) {
      wgrad_chunks(B, C, wgrad_planes_per_iter(B, H, W, K, levels), kWgradResident, &bchunk, &nchunk);
      floats = static_cast<size_t>(nchunk) * C * ((1 + 4 * levels) * K * K + 1);
    } else {      // partial sums, then the pyramids of x and of grad_out
      nchunk = stream_chunks(B, C, H, W);
      floats = round_up64(static_cast<size_t>(nchunk) * C * ((1 + 4 * levels) * K * K + 1)) +
               2 * make_stream2d(B, C, H, W, levels).floats;
    }
    if (mfloats > floats) floats = mfloats;
    floats = round_up64(floats) + static_cast<size_t>(C);      // one ticket word per channel behind the records
  } else {
    // the dtype is not an argument here: size for the larger of the two (fp32 tensors take
    // three split tables) whenever either could run on the matrix-core kernels
    size_t mf = 0;
    for (int dt : {WTCONV_F32, WTCONV_BF16}) {
      const Mfma2dQuery q = mfma2d_query(B, C, H, W, K, levels, dt);
      if (q.ok && q.ws_bytes > mf) mf = q.ws_bytes;
    }
    floats = fold_floats(C, 4, levels, K * K);
    if (!plane_fits_lds(B, C, H, W, K, levels)) floats = round_up64(floats) + make_stream2d(B, C, H, W, levels).floats;
    if (mf > floats * sizeof(float)) floats = (mf + 3) / 4;
  }
  return (floats * sizeof(float) + 255) / 256 * 256;
}

int wtconv2d_forward(const void* x, void* out, const wtconv_params* params, int B, int C, int H, int W, int K,
                     int levels, int dtype, int param_dtype, void* workspace, size_t workspace_bytes,
                     void* stream) {
  return plane2d_pass("wtconv2d_forward", x, out, params, B, C, H, W, K, levels, dtype, param_dtype, workspace,
                      workspace_bytes, stream, 0);
}

size_t wtconv_static_scratch_bytes(void) { return kStaticScratchBytes; }

int wtconv2d_forward_static(const void* x, void* out, const wtconv_params* params, int B, int C, int H, int W,
                            int K, int levels, int dtype, int param_dtype, void* stream) {
  const char* fn = "wtconv2d_forward_static";
  const size_t need = wtconv2d_workspace_bytes(B, C, H, W, K, levels, WTCONV_PASS_FORWARD);
  if (need > kStaticScratchBytes)
    return fail(WTCONV_E_UNSUPPORTED,
                "%s: this shape needs %zu B of scratch, the static buffer holds %zu B; use wtconv2d_forward with a "
                "caller-supplied workspace", fn, need, kStaticScratchBytes);
  void* ptr = nullptr;
  if (int e = static_scratch(fn, &ptr)) return e;
  return plane2d_pass(fn, x, out, params, B, C, H, W, K, levels, dtype, param_dtype, ptr, kStaticScratchBytes,
                      stream, 0);
}

int wtconv2d_backward_input(const void* grad_out, void* grad_x, const wtconv_params* params, int B, int C,
                            int H, int W, int K, int levels, int dtype, int param_dtype, void* workspace,
                            size_t workspace_bytes, void* stream) {
  return plane2d_pass("wtconv2d_backward_input", grad_out, grad_x, params, B, C, H, W, K, levels, dtype,
                      param_dtype, workspace, workspace_bytes, stream, 1);
}

// Where the parameter-gradient pass of a plane-resident shape keeps its channel tickets in the workspace.
static unsigned* wgrad2d_tickets(void* workspace, int B, int C, int H, int W, int K, int L) {
  const size_t need = wtconv2d_workspace_bytes(B, C, H, W, K, L, WTCONV_PASS_BACKWARD_PARAMS);
  return reinterpret_cast<unsigned*>(static_cast<char*>(workspace) + need) - C;
}

// have_g_pyramid (level-by-level path only): the pyramid of grad_out is in its place in the workspace already.
// tickets_zeroed (plane-resident paths only): an earlier kernel on the stream has cleared the channel tickets.
static int backward_params2d(const char* fn, const void* x, const void* grad_out, const wtconv_params* params,
                             const wtconv_param_grads* grads, int B, int C, int H, int W, int K, int levels,
                             int dtype, int param_dtype, void* workspace, size_t workspace_bytes,
                             void* stream_, bool have_g_pyramid, bool tickets_zeroed = false) {
  const int L = levels;
  if (int e = check_common(fn, params, B, C, K, L, dtype, param_dtype)) return e;
  if (H <= 0 || W <= 0) return fail(WTCONV_E_ARG, "%s: spatial size must be positive (got %dx%d)", fn, H, W);
  if (static_cast<long long>(H) * W > kMaxPlaneElems)   // 32-bit offsets inside a plane and its four stacked sub-bands
    return fail(WTCONV_E_UNSUPPORTED, "%s: a plane of %dx%d exceeds 2^28 elements", fn, H, W);
  if (x == nullptr || grad_out == nullptr || grads == nullptr) return fail(WTCONV_E_ARG, "%s: null tensor pointer", fn);
  if (grads->base_weight == nullptr || grads->base_scale == nullptr ||
      (params->base_bias != nullptr && grads->base_bias == nullptr))
    return fail(WTCONV_E_ARG, "%s: null gradient pointer", fn);
  for (int l = 0; l < L; ++l)
    if (grads->wt_weight[l] == nullptr || grads->wt_scale[l] == nullptr)
      return fail(WTCONV_E_ARG, "%s: null gradient pointer at level %d", fn, l);
  const size_t esz = dtype == WTCONV_F32 ? 4 : 2;
  if ((reinterpret_cast<uintptr_t>(x) % esz) || (reinterpret_cast<uintptr_t>(grad_out) % esz))
    return fail(WTCONV_E_ARG, "%s: tensor pointer not aligned to its element size", fn);
  const size_t need = wtconv2d_workspace_bytes(B, C, H, W, K, L, WTCONV_PASS_BACKWARD_PARAMS);
  if (workspace == nullptr || workspace_bytes < need)
    return fail(WTCONV_E_WORKSPACE, "%s: workspace of %zu B needed, %zu given", fn, need, workspace_bytes);
  if (static_cast<long long>(B) * C > 0x7fffffffLL / 4)
    return fail(WTCONV_E_UNSUPPORTED, "%s: batch*channels = %lld is too large", fn, static_cast<long long>(B) * C);
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  int bchunk, nchunk;
  float* partial = static_cast<float*>(workspace);
  int e;
  const Mfma2dWgradQuery mq = mfma2d_wgrad_query(B, C, H, W, K, L, dtype);
  const bool resident = mq.ok || wgrad_fits_lds(B, C, H, W, K, L);
  // The plane-resident first-stage kernels finish their channels themselves (last workgroup of a channel): one ticket
  // word per channel at the end of the workspace, cleared by a small launch of its own.
  FinishArgs fin = {};
  if (resident) {
    fin.tickets = wgrad2d_tickets(workspace, B, C, H, W, K, L);
    fin.prm = to_table(params, L);
    fin.pdtype = param_dtype;
    fin.gt = to_grad_table(grads, L);
    if (!tickets_zeroed) {
      WT_LAUNCH(zero_tickets_kernel, dim3((C + 255) / 256), dim3(256), 0, stream, fin.tickets, C);
      if (int ze = check_launch("zero_tickets_kernel")) return ze;
    }
  }
  if (mq.ok) {
    nchunk = mq.nchunk;
    e = mfma2d_wgrad_pass(fn, x, grad_out, partial, B, C, H, W, K, L, fin, stream);
  } else if (resident) {
    const int pb = wgrad_planes_per_iter(B, H, W, K, L);
    Plan2D pl = make_plan2d(B, C, H, W, K, L, true, 512, esz, x, grad_out, nullptr, pb);
    finish_wgrad_plan(&pl, K);
    wgrad_chunks(B, C, pb, kWgradResident, &bchunk, &nchunk);
    e = dtype == WTCONV_F32   ? run_wgrad2d_static<float>(K, L, x, grad_out, partial, pl, B, bchunk, nchunk, fin, stream)
        : dtype == WTCONV_F16 ? run_wgrad2d_static<f16_t>(K, L, x, grad_out, partial, pl, B, bchunk, nchunk, fin, stream)
                              : 1;
    if (e == 1)
      e = WT_BY_DTYPE(dtype, run_wgrad2d_k<T_>(K, L, x, grad_out, partial, pl, B, bchunk, nchunk, fin, stream));
  } else {
    const Stream2D sp = make_stream2d(B, C, H, W, L);
    nchunk = stream_chunks(B, C, H, W);
    if (nchunk > 65535 || C > 0x7fffffff / 4) return fail(WTCONV_E_UNSUPPORTED, "%s: too many chunks (%d)", fn, nchunk);
    float* pyr_x = partial + round_up64(static_cast<size_t>(nchunk) * C * ((1 + 4 * L) * K * K + 1));
    float* pyr_g = pyr_x + sp.floats;
    e = WT_BY_DTYPE(dtype, run_stream2d_wgrad_k<T_>(K, x, grad_out, partial, pyr_x, pyr_g, sp, B, nchunk, stream,
                                                    have_g_pyramid));
  }
  if (e || resident) return e;
  const GradTable gt = to_grad_table(grads, L);
  const int nrec = (1 + 4 * L) * K * K + 1;
  WT_LAUNCH(wgrad_finish_kernel, dim3(C), dim3(finish_threads(nrec)), static_cast<size_t>(nrec) * sizeof(float),
            stream, partial, nchunk, to_table(params, L), param_dtype, gt, C, 4, L, K * K);
  return check_launch("wgrad_finish_kernel");
}

int wtconv2d_backward_params(const void* x, const void* grad_out, const wtconv_params* params,
                             const wtconv_param_grads* grads, int B, int C, int H, int W, int K, int levels,
                             int dtype, int param_dtype, void* workspace, size_t workspace_bytes,
                             void* stream) {
  return backward_params2d("wtconv2d_backward_params", x, grad_out, params, grads, B, C, H, W, K, levels, dtype,
                           param_dtype, workspace, workspace_bytes, stream, false);
}

int wtconv2d_backward(const void* x, const void* grad_out, void* grad_x, const wtconv_params* params,
                      const wtconv_param_grads* grads, int B, int C, int H, int W, int K, int levels, int dtype,
                      int param_dtype, void* workspace, size_t workspace_bytes, void* stream) {
  // Planes beyond LDS (both passes level by level): the pyramid of grad_out is built once, in the place the
  // parameter-gradient pass keeps it, and serves both passes; the folded parameters of the input-gradient pass sit
  // where the pyramid of x goes afterwards.
  const bool sizes_ok = B > 0 && C > 0 && H > 0 && W > 0 && K >= 1 && K % 2 == 1 && K <= wtconv_max_kernel_size() &&
                        levels >= 2 && levels <= kMaxLevels && static_cast<long long>(H) * W <= kMaxPlaneElems;
  if (sizes_ok && !mfma2d_query(B, C, H, W, K, levels, dtype).ok && !plane_fits_lds(B, C, H, W, K, levels) &&
      !mfma2d_wgrad_query(B, C, H, W, K, levels, dtype).ok && !wgrad_fits_lds(B, C, H, W, K, levels)) {
    const size_t need = wtconv2d_workspace_bytes(B, C, H, W, K, levels, WTCONV_PASS_BACKWARD);
    if (workspace == nullptr || workspace_bytes < need)
      return fail(WTCONV_E_WORKSPACE, "wtconv2d_backward: workspace of %zu B needed, %zu given", need, workspace_bytes);
    const Stream2D sp = make_stream2d(B, C, H, W, levels);
    const int nchunk = stream_chunks(B, C, H, W);
    float* partial = static_cast<float*>(workspace);
    float* pyr_x = partial + round_up64(static_cast<size_t>(nchunk) * C * ((1 + 4 * levels) * K * K + 1));
    float* pyr_g = pyr_x + sp.floats;
    if (fold_floats(C, 4, levels, K * K) <= sp.floats) {
      if (int e = plane2d_pass("wtconv2d_backward", grad_out, grad_x, params, B, C, H, W, K, levels, dtype, param_dtype,
                               workspace, workspace_bytes, stream, 1, pyr_g, pyr_x))
        return e;
      return backward_params2d("wtconv2d_backward", x, grad_out, params, grads, B, C, H, W, K, levels, dtype,
                               param_dtype, workspace, workspace_bytes, stream, true);
    }
  }
  // Otherwise the two passes run one after the other on the stream and share the workspace.  Plane-resident shapes:
  // the input-gradient pass clears the channel tickets of the parameter-gradient pass on its way (one launch fewer),
  // where they lie beyond the folded parameters that it keeps at the start of the workspace.
  if (sizes_ok && workspace != nullptr &&
      workspace_bytes >= wtconv2d_workspace_bytes(B, C, H, W, K, levels, WTCONV_PASS_BACKWARD) &&
      (mfma2d_query(B, C, H, W, K, levels, dtype).ok || plane_fits_lds(B, C, H, W, K, levels)) &&
      (mfma2d_wgrad_query(B, C, H, W, K, levels, dtype).ok || wgrad_fits_lds(B, C, H, W, K, levels))) {
    unsigned* tickets = wgrad2d_tickets(workspace, B, C, H, W, K, levels);
    const char* fold_end = static_cast<const char*>(workspace) + fold_floats(C, 4, levels, K * K) * sizeof(float);
    if (reinterpret_cast<const char*>(tickets) >= fold_end) {
      if (int e = plane2d_pass("wtconv2d_backward", grad_out, grad_x, params, B, C, H, W, K, levels, dtype, param_dtype,
                               workspace, workspace_bytes, stream, 1, nullptr, nullptr, tickets))
        return e;
      return backward_params2d("wtconv2d_backward", x, grad_out, params, grads, B, C, H, W, K, levels, dtype,
                               param_dtype, workspace, workspace_bytes, stream, false, true);
    }
  }
  if (int e = wtconv2d_backward_input(grad_out, grad_x, params, B, C, H, W, K, levels, dtype, param_dtype, workspace,
                                      workspace_bytes, stream))
    return e;
  return wtconv2d_backward_params(x, grad_out, params, grads, B, C, H, W, K, levels, dtype, param_dtype, workspace,
                                  workspace_bytes, stream);
}

size_t wtconv1d_workspace_bytes(int B, int C, int N, int K, int levels, int pass) {
  if (pass == WTCONV_PASS_BACKWARD) {
    const size_t a = wtconv1d_workspace_bytes(B, C, N, K, levels, WTCONV_PASS_BACKWARD_INPUT);
    const size_t b = wtconv1d_workspace_bytes(B, C, N, K, levels, WTCONV_PASS_BACKWARD_PARAMS);
    return a > b ? a : b;
  }
  if (B <= 0 || C <= 0 || N <= 0 || K <= 0 || levels <= 0 || levels > kMaxLevels) return 0;
  size_t floats;
  if (pass == WTCONV_PASS_BACKWARD_PARAMS) {
    const Plan1D pl = make_plan1d(C, N, K, levels, true, 4, nullptr, nullptr, nullptr);
    int per_chunk, nchunk;
    Row1DShape sh = {};
    if (row1d_shape(N, K, levels, kRow1dMaxLanes, &sh))
      row1d_chunks(B, C, row1d_two_region_per_cu(K, levels, sh), &per_chunk, &nchunk);
    else
      wgrad_chunks1d(B, C, pl.ntiles, &per_chunk, &nchunk);
    // partial sums, then one ticket word per channel (fused backward kernel)
    floats = round_up64(static_cast<size_t>(nchunk) * C * ((1 + 2 * levels) * K + 1)) + static_cast<size_t>(C);
  } else {
    floats = fold_floats(C, 2, levels, K);
  }
  return (floats * sizeof(float) + 255) / 256 * 256;
}

int wtconv1d_forward(const void* x, void* out, const wtconv_params* params, int B, int C, int N, int K,
                     int levels, int dtype, int param_dtype, void* workspace, size_t workspace_bytes,
                     void* stream) {
  return tile1d_pass("wtconv1d_forward", x, out, params, B, C, N, K, levels, dtype, param_dtype, workspace,
                     workspace_bytes, stream, 0);
}

int wtconv1d_backward_input(const void* grad_out, void* grad_x, const wtconv_params* params, int B, int C,
                            int N, int K, int levels, int dtype, int param_dtype, void* workspace,
                            size_t workspace_bytes, void* stream) {
  return tile1d_pass("wtconv1d_backward_input", grad_out, grad_x, params, B, C, N, K, levels, dtype,
                     param_dtype, workspace, workspace_bytes, stream, 1);
}

int wtconv1d_backward_params(const void* x, const void* grad_out, const wtconv_params* params,
                             const wtconv_param_grads* grads, int B, int C, int N, int K, int levels,
                             int dtype, int param_dtype, void* workspace, size_t workspace_bytes,
                             void* stream_) {
  const char* fn = "wtconv1d_backward_params";
  const int L = levels;
  if (int e = check_common(fn, params, B, C, K, L, dtype, param_dtype)) return e;
  if (N <= 0) return fail(WTCONV_E_ARG, "%s: length must be positive (got %d)", fn, N);
  if (x == nullptr || grad_out == nullptr || grads == nullptr) return fail(WTCONV_E_ARG, "%s: null tensor pointer", fn);
  if (grads->base_weight == nullptr || grads->base_scale == nullptr ||
      (params->base_bias != nullptr && grads->base_bias == nullptr))
    return fail(WTCONV_E_ARG, "%s: null gradient pointer", fn);
  for (int l = 0; l < L; ++l)
    if (grads->wt_weight[l] == nullptr || grads->wt_scale[l] == nullptr)
      return fail(WTCONV_E_ARG, "%s: null gradient pointer at level %d", fn, l);
  const size_t esz = dtype == WTCONV_F32 ? 4 : 2;
  if ((reinterpret_cast<uintptr_t>(x) % esz) || (reinterpret_cast<uintptr_t>(grad_out) % esz))
    return fail(WTCONV_E_ARG, "%s: tensor pointer not aligned to its element size", fn);
  const Plan1D pl = make_plan1d(C, N, K, L, true, esz, x, grad_out, nullptr);
  const size_t need = wtconv1d_workspace_bytes(B, C, N, K, L, WTCONV_PASS_BACKWARD_PARAMS);
  if (workspace == nullptr || workspace_bytes < need)
    return fail(WTCONV_E_WORKSPACE, "%s: workspace of %zu B needed, %zu given", fn, need, workspace_bytes);
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  int per_chunk, nchunk;
  Row1DShape sh = {};
  const bool row_resident = row1d_shape(N, K, L, kRow1dMaxLanes, &sh);
  if (row_resident)
    row1d_chunks(B, C, row1d_two_region_per_cu(K, L, sh), &per_chunk, &nchunk);
  else
    wgrad_chunks1d(B, C, pl.ntiles, &per_chunk, &nchunk);
  if (nchunk > 65535) return fail(WTCONV_E_UNSUPPORTED, "%s: too many chunks (%d)", fn, nchunk);
  float* partial = static_cast<float*>(workspace);
  int e;
  if (row_resident) {
    const Row1D rp = make_row1d(C, N, sh.nl, esz, x, grad_out);
    e = WT_BY_DTYPE(dtype, run_row1d_wgrad_kl<T_>(K, L, sh.S, x, grad_out, partial, rp, B, sh.block, per_chunk, nchunk,
                                                  stream));
  } else {
    e = WT_BY_DTYPE(dtype, run_wgrad1d_k<T_>(K, L, x, grad_out, partial, pl, B, per_chunk, nchunk, stream));
  }
  if (e) return e;
  GradTable gt = {};
  gt.base_weight = grads->base_weight;
  gt.base_bias = grads->base_bias;
  gt.base_scale = grads->base_scale;
  for (int l = 0; l < L; ++l) { gt.wt_weight[l] = grads->wt_weight[l]; gt.wt_scale[l] = grads->wt_scale[l]; }
  const int nrec = (1 + 2 * L) * K + 1;
  WT_LAUNCH(wgrad_finish_kernel, dim3(C), dim3(finish_threads(nrec)), static_cast<size_t>(nrec) * sizeof(float),
            stream, partial, nchunk, to_table(params, L), param_dtype, gt, C, 2, L, K);
  return check_launch("wgrad_finish_kernel");
}

int wtconv1d_backward(const void* x, const void* grad_out, void* grad_x, const wtconv_params* params,
                      const wtconv_param_grads* grads, int B, int C, int N, int K, int levels, int dtype,
                      int param_dtype, void* workspace, size_t workspace_bytes, void* stream) {
  const char* fn = "wtconv1d_backward";
  // rows that the register-resident kernels take run the whole backward pass as one kernel -- with the lanes, chunks
  // and workspace layout of the separate parameter-gradient pass, so the two share wtconv1d_workspace_bytes
  Row1DShape sh = {};
  if (K >= 1 && levels >= 1 && levels <= kMaxLevels && row1d_shape(N, K, levels, kRow1dMaxLanes, &sh) &&
      sh.block <= kRow1dBwdMaxLanes && row1d_bwd_built(K, levels, sh.S)) {
    const int L = levels;
    if (int e = check_common(fn, params, B, C, K, L, dtype, param_dtype)) return e;
    if (x == nullptr || grad_out == nullptr || grad_x == nullptr) return fail(WTCONV_E_ARG, "%s: null tensor pointer", fn);
    if (int e = check_grad_table(fn, params, grads, L)) return e;
    const size_t esz = dtype == WTCONV_F32 ? 4 : 2;
    if ((reinterpret_cast<uintptr_t>(x) % esz) || (reinterpret_cast<uintptr_t>(grad_out) % esz) ||
        (reinterpret_cast<uintptr_t>(grad_x) % esz))
      return fail(WTCONV_E_ARG, "%s: tensor pointer not aligned to its element size", fn);
    const size_t need = wtconv1d_workspace_bytes(B, C, N, K, L, WTCONV_PASS_BACKWARD);
    if (workspace == nullptr || workspace_bytes < need)
      return fail(WTCONV_E_WORKSPACE, "%s: workspace of %zu B needed, %zu given", fn, need, workspace_bytes);
    if (reinterpret_cast<uintptr_t>(workspace) % 4)
      return fail(WTCONV_E_ARG, "%s: workspace not aligned", fn);
    int per_chunk, nchunk;
    row1d_chunks(B, C, row1d_two_region_per_cu(K, L, sh), &per_chunk, &nchunk);
    if (nchunk > 65535) return fail(WTCONV_E_UNSUPPORTED, "%s: too many chunks (%d)", fn, nchunk);
    float* partial = static_cast<float*>(workspace);
    unsigned* tickets = reinterpret_cast<unsigned*>(partial + round_up64(static_cast<size_t>(nchunk) * C * ((1 + 2 * L) * K + 1)));
    Row1D rp = make_row1d(C, N, sh.nl, esz, x, grad_out);
    rp.vec_ok = rp.vec_ok && (reinterpret_cast<uintptr_t>(grad_x) & 15u) == 0;
    const GradTable gt = to_grad_table(grads, L);
    return WT_BY_DTYPE(dtype, run_row1d_bwd_kl<T_>(K, L, sh.S, x, grad_out, grad_x, partial, tickets, params, param_dtype,
                                                    gt, rp, B, sh.block, per_chunk, nchunk,
                                                    static_cast<hipStream_t>(stream)));
  }
  if (int e = wtconv1d_backward_input(grad_out, grad_x, params, B, C, N, K, levels, dtype, param_dtype, workspace,
                                      workspace_bytes, stream))
    return e;
  return wtconv1d_backward_params(x, grad_out, params, grads, B, C, N, K, levels, dtype, param_dtype, workspace,
                                  workspace_bytes, stream);
}

}  // extern "C"
