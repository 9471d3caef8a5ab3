// Host side of the matrix-core 2-D path: LDS planning, dispatch and launches of
// kernels2d_mfma.h.  Allocates nothing, never synchronises.
#include <stdlib.h>
#include <string.h>

#include "common.h"
#include "host_util.h"
#include "kernels2d_mfma.h"
#include "kernels2d_mfma_wgrad.h"
#include "mfma2d.h"

namespace wt {

namespace {

inline int ceil_div(int a, int b) { return (a + b - 1) / b; }

// LDS layout and unit geometry for `pb` planes per unit; false if the kernel cannot index it.
bool make_mplan(int B, int C, int H, int W, int L, int NS, int pb, MPlan* out) {
  if (!make_mplan_geometry(H, W, L, NS, pb, out)) return false;
  out->B = B; out->C = C;
  out->upc = ceil_div(B, pb);
  out->bq = B / out->upc;
  out->br = B % out->upc;
  if (static_cast<long long>(C) * out->upc > 0x7fffffffLL) return false;
  out->nunits = C * out->upc;
  if (static_cast<long long>(pb) * C * H * W > 0x7fffffffLL) return false;
  return true;
}

// Which tensors take the matrix-core kernels (environment variable WTCONV_MFMA, read once):
// 0 none; 1 bf16 tensors (the default); 2 bf16 and fp32 tensors, the latter split into three bf16
// planes -- exact to fp32 rounding, but slower than the vector-ALU kernels on the shapes measured.
int mfma_mode() {
  static const int mode = [] {
    const char* e = getenv("WTCONV_MFMA");
    return e ? atoi(e) : 1;
  }();
  return mode;
}

size_t lds_budget() {
#ifdef WT_EMULATE
  if (const char* e = getenv("WT_EMU_LDS_LIMIT")) return static_cast<size_t>(atol(e));
#endif
  return kLdsLimitBytes;
}

// Planes per unit: as many as keep every thread's share at one 4x4 block, shrunk until a
// workgroup's LDS leaves room for several workgroups per CU.
bool choose_mplan_uncached(int B, int C, int H, int W, int L, int NS, MPlan* out, int* nbl);

// Plans are pure functions of the shape; the search behind them (candidate plane counts, checked
// reciprocals) is too slow to repeat on every call, so results are kept per thread.
struct PlanKey {
  int B, C, H, W, L, NS;
  bool operator==(const PlanKey& o) const { return B == o.B && C == o.C && H == o.H && W == o.W && L == o.L && NS == o.NS; }
};
struct PlanKeyHash {
  size_t operator()(const PlanKey& k) const {
    size_t h = 1469598103934665603ull;
    for (int v : {k.B, k.C, k.H, k.W, k.L, k.NS}) h = (h ^ static_cast<size_t>(v)) * 1099511628211ull;
    return h;
  }
};
struct PlanVal { bool ok; MPlan pl; int nbl; };

bool choose_mplan(int B, int C, int H, int W, int L, int NS, MPlan* out, int* nbl) {
  static thread_local std::unordered_map<PlanKey, PlanVal, PlanKeyHash> cache;
  const PlanKey key = {B, C, H, W, L, NS};
  auto it = cache.find(key);
  if (it == cache.end()) {
    if (cache.size() > 4096) cache.clear();
    PlanVal v = {};
    v.ok = choose_mplan_uncached(B, C, H, W, L, NS, &v.pl, &v.nbl);
    it = cache.emplace(key, v).first;
  }
  if (it->second.ok) { *out = it->second.pl; *nbl = it->second.nbl; }
  return it->second.ok;
}

bool choose_mplan_uncached(int B, int C, int H, int W, int L, int NS, MPlan* out, int* nbl) {
  const int bpp0 = ceil_div(H, 4) * ceil_div(W, 4);
  int pb = kMfmaBlock / bpp0;
  if (pb < 1) pb = 1;
  if (pb > B) pb = B;
  // Four workgroups per CU (40 KB each) where the planes allow it; three (53 KB) if that puts
  // clearly more threads to work in the load phase of planes of 14 x 14 and larger (measured, bf16,
  // stage shapes: 28 x 28 planes 48 -> 44 us with 4 instead of 3 planes; 7 x 7 planes are faster
  // with 27 planes and four workgroups than with 32 and three).
  const size_t want = NS == 1 ? 40 * 1024 : 80 * 1024, relaxed = NS == 1 ? 53 * 1024 : 80 * 1024;
  const int pb_max = pb;
  MPlan pl;
  for (;; --pb) {
    if (!make_mplan(B, C, H, W, L, NS, pb, &pl)) return false;
    if (static_cast<size_t>(pl.lds_bytes) <= want || pb == 1) break;
  }
  if (bpp0 >= 16 && pl.nblk[0] * 10 < kMfmaBlock * 6) {
    for (int p2 = pb_max; p2 > pb; --p2) {
      MPlan alt;
      if (B % p2 == 0 && make_mplan(B, C, H, W, L, NS, p2, &alt) && static_cast<size_t>(alt.lds_bytes) <= relaxed) {
        pl = alt;
        pb = p2;
        break;
      }
    }
  }
  if (static_cast<size_t>(pl.lds_bytes) > lds_budget()) return false;
  const int per_thread = ceil_div(pl.nblk[0], kMfmaBlock);
  if (per_thread > 4) return false;
  *nbl = per_thread <= 1 ? 1 : (per_thread == 2 ? 2 : 4);
  *out = pl;
  return true;
}

// Parameter table and folding options of a pass.
struct MfmaArgs {
  ParamTable prm;
  int pdtype, K, flip, use_bias;
  unsigned* zero_words;
  int nzero;
};

template <typename T, int NS, int NBL, bool VEC, typename Geo>
int launch_mfma(const void* x, void* out, const MfmaArgs& a, const MPlan& pl, hipStream_t stream) {
  auto kern = wt2d_mfma_kernel<T, NS, NBL, VEC, NS == 1, Geo>;
  const size_t lds = static_cast<size_t>(pl.lds_bytes);
  if (int e = allow_lds(kern, lds)) return e;
  int nwg = compute_units() * resident_per_cu(kern, kMfmaBlock, lds);
  if (nwg > pl.nunits) nwg = pl.nunits;
  WT_LAUNCH(kern, dim3(nwg), dim3(kMfmaBlock), lds, stream, static_cast<const T*>(x), static_cast<T*>(out), a.prm,
            a.pdtype, a.K, a.flip, a.use_bias, pl, a.zero_words, a.nzero);
  return check_launch("wt2d_mfma_kernel");
}

template <typename T, int NS, int NBL>
int launch_mfma_vec(bool vec, const void* x, void* out, const MfmaArgs& a, const MPlan& pl,
                    hipStream_t stream) {
  return vec ? launch_mfma<T, NS, NBL, true, GeoRuntime>(x, out, a, pl, stream)
             : launch_mfma<T, NS, NBL, false, GeoRuntime>(x, out, a, pl, stream);
}

// The WTConvNeXt stage shapes (56/28/14/7 squares; 3/3/2/2 levels as single layers, 5/4/3/2 in the
// model) have kernels whose whole LDS layout is a compile-time constant.
template <typename T, int NS, int H, int L, int PB, bool VEC>
bool try_static(bool vec, const void* x, void* out, const MfmaArgs& a, const MPlan& pl,
                hipStream_t stream, int* rc) {
  if (pl.H != H || pl.W != H || pl.L != L || pl.pb != PB || vec != VEC) return false;
  *rc = launch_mfma<T, NS, 1, VEC, GeoStatic<H, H, L, PB>>(x, out, a, pl, stream);
  return true;
}

template <typename T, int NS>
int launch_mfma_nbl(int nbl, bool vec, const void* x, void* out, const MfmaArgs& a, const MPlan& pl,
                    hipStream_t stream) {
#ifndef WT_EMULATE
  int rc = 0;
#define WT_TRY(H_, L_, PB_, VEC_) \
  if (try_static<T, NS, H_, L_, PB_, VEC_>(vec, x, out, a, pl, stream, &rc)) return rc;
  if constexpr (NS == 1) {
    WT_TRY(56, 3, 1, true) WT_TRY(28, 3, 4, true) WT_TRY(14, 2, 11, false) WT_TRY(7, 2, 29, false)
    WT_TRY(56, 5, 1, true) WT_TRY(28, 4, 4, true) WT_TRY(14, 3, 9, false)
  } else {
    WT_TRY(56, 3, 1, true) WT_TRY(28, 3, 2, true) WT_TRY(14, 2, 9, false) WT_TRY(7, 2, 21, false)
  }
#undef WT_TRY
#endif
  switch (nbl) {
    case 1: return launch_mfma_vec<T, NS, 1>(vec, x, out, a, pl, stream);
    case 2: return launch_mfma_vec<T, NS, 2>(vec, x, out, a, pl, stream);
    default: return launch_mfma_vec<T, NS, 4>(vec, x, out, a, pl, stream);
  }
}

}  // namespace

Mfma2dQuery mfma2d_query(int B, int C, int H, int W, int K, int L, int dtype) {
  Mfma2dQuery r = {false, 0};
  const int mode = mfma_mode();
  if (mode <= 0 || K > 5 || L < 1 || L > kMaxLevels) return r;
  if (dtype != WTCONV_BF16 && !(dtype == WTCONV_F32 && mode >= 2)) return r;
  const int NS = dtype == WTCONV_F32 ? 3 : 1;
  MPlan pl;
  int nbl;
  if (!choose_mplan(B, C, H, W, L, NS, &pl, &nbl)) return r;
  r.ok = true;
  r.ws_bytes = 0;       // the kernel folds the parameters of a channel itself
  return r;
}

int mfma2d_pass(const char* fn, const void* x, void* out, const wtconv_params* params, int B, int C, int H, int W,
                int K, int L, int dtype, int pdtype, hipStream_t stream, int flip, unsigned* zero_words, int nzero) {
  const int NS = dtype == WTCONV_F32 ? 3 : 1;
  MPlan pl;
  int nbl;
  if (!choose_mplan(B, C, H, W, L, NS, &pl, &nbl))
    return fail(WTCONV_E_UNSUPPORTED, "%s: shape not covered by the matrix-core kernels", fn);
  const MfmaArgs a = {to_table(params, L), pdtype, K, flip, flip ? 0 : 1, zero_words, zero_words != nullptr ? nzero : 0};
  const size_t esz = dtype == WTCONV_F32 ? 4 : 2;
  const uintptr_t mask = 4 * esz - 1;
  const bool vec = (W % 4 == 0) && (reinterpret_cast<uintptr_t>(x) & mask) == 0 &&
                   (reinterpret_cast<uintptr_t>(out) & mask) == 0;
  return dtype == WTCONV_F32 ? launch_mfma_nbl<float, 3>(nbl, vec, x, out, a, pl, stream)
                             : launch_mfma_nbl<bf16_t, 1>(nbl, vec, x, out, a, pl, stream);
}

// ---- parameter gradients ---------------------------------------------------------------------
namespace {

constexpr int kWgradLdsPair = 80 * 1024;      // two workgroups of four waves per CU below this, else one of eight waves
constexpr int kWgradLdsTriple = 53 * 1024;    // three workgroups per CU below this

struct WKey {
  int B, C, H, W, L;
  bool operator==(const WKey& o) const { return B == o.B && C == o.C && H == o.H && W == o.W && L == o.L; }
};
struct WKeyHash {
  size_t operator()(const WKey& k) const {
    size_t h = 1469598103934665603ull;
    for (int v : {k.B, k.C, k.H, k.W, k.L}) h = (h ^ static_cast<size_t>(v)) * 1099511628211ull;
    return h;
  }
};
struct WVal { bool ok; WPlan pl; int nw, compact, bchunk, nchunk; };

// Planes per unit: up to one 4x4 block per thread of four waves.  Small planes, of which at least two fit a third
// of the LDS, run as three workgroups per CU (a unit's phases are short and wait on its loads, so a third
// workgroup in another phase pays more than larger units: 7 x 7 planes 38 -> 28 us, 14 x 14 34 -> 29 us, 28 x 28
// 57 -> 50 us per launch at batch 128); otherwise as many planes as leave room for two workgroups per CU; a single
// plane beyond that runs as one workgroup of eight waves per CU.
bool choose_wplan(int B, int C, int H, int W, int L, WVal* v) {
  const int bpp0 = ceil_div(H, 4) * ceil_div(W, 4);
  int pb = kMfmaBlock / bpp0;
  if (pb < 1 || W > 64) return false;
  if (pb > B) pb = B;
  if (static_cast<long long>(pb) * C * H * W > 0x7fffffffLL) return false;
  WPlan pl;
  bool compact = false;
  const int pb_max = pb;
  for (;; --pb) {
    if (!make_wplan_geometry(H, W, L, pb, 512, false, &pl)) return false;
    if (pl.lds_bytes <= kWgradLdsTriple || pb == 1) break;
  }
  if (pl.lds_bytes > kWgradLdsTriple || (pb < 2 && pb_max >= 2)) {
    for (pb = pb_max;; --pb) {
      if (!make_wplan_geometry(H, W, L, pb, 512, false, &pl)) return false;
      if (pl.lds_bytes <= kWgradLdsPair || pb == 1) break;
    }
  }
  if (pl.lds_bytes > kWgradLdsPair) {
    WPlan cp;
    if (make_wplan_geometry(H, W, L, pb, 512, true, &cp) && cp.lds_bytes <= kWgradLdsPair) { pl = cp; compact = true; }
  }
  if (static_cast<size_t>(pl.lds_bytes) > lds_budget()) return false;
  pl.B = B; pl.C = C;
  v->pl = pl;
  v->compact = compact;
  v->nw = pl.lds_bytes <= kWgradLdsPair ? 4 : 8;
  const int per_cu = v->nw == 8 ? 1 : (pl.lds_bytes <= kWgradLdsTriple ? 3 : 2);
  wgrad_chunks(B, C, pb, compute_units() * per_cu, &v->bchunk, &v->nchunk);
  return true;
}

// Shape-only part of the plan (pointer alignment is applied per call).
const WVal& wplan_cached(int B, int C, int H, int W, int L) {
  static thread_local std::unordered_map<WKey, WVal, WKeyHash> cache;
  const WKey key = {B, C, H, W, L};
  auto it = cache.find(key);
  if (it == cache.end()) {
    if (cache.size() > 4096) cache.clear();
    WVal v = {};
    v.ok = choose_wplan(B, C, H, W, L, &v);
    it = cache.emplace(key, v).first;
  }
  return it->second;
}

struct WgradArgs { const void* x; const void* g; float* partial; int K, bchunk, nchunk; FinishArgs fin; };

template <int L, int NW, bool VEC, typename Geo>
int launch_wgrad(const WgradArgs& a, const WPlan& pl, hipStream_t stream) {
  auto kern = wt2d_mfma_wgrad_kernel<L, NW, VEC, Geo>;
  const size_t lds = static_cast<size_t>(pl.lds_bytes);
  if (int e = allow_lds(kern, lds)) return e;
  WT_LAUNCH(kern, dim3(pl.C, a.nchunk), dim3(NW * 64), lds, stream, static_cast<const bf16_t*>(a.x),
            static_cast<const bf16_t*>(a.g), a.partial, pl, a.K, a.bchunk, a.fin);
  return check_launch("wt2d_mfma_wgrad_kernel");
}

template <int L>
int launch_wgrad_l(int nw, bool compact, bool vec, const WgradArgs& a, const WPlan& pl, hipStream_t stream) {
#ifndef WT_EMULATE
  // plane shapes of the WTConvNeXt stages: geometry as a compile-time constant
#define WT_TRY(H_, L_, PB_, NW_, CMP_) \
  if (L == L_ && pl.H == H_ && pl.W == H_ && pl.pb == PB_ && nw == NW_ && compact == CMP_ && vec == (H_ % 4 == 0)) \
    return launch_wgrad<L_, NW_, H_ % 4 == 0, WGeoStatic<H_, H_, L_, PB_, 512, CMP_>>(a, pl, stream);
  WT_TRY(56, 3, 1, 4, true) WT_TRY(28, 3, 2, 4, false) WT_TRY(14, 2, 7, 4, false) WT_TRY(7, 2, 16, 4, false)
  WT_TRY(56, 5, 1, 8, false) WT_TRY(28, 4, 2, 4, false) WT_TRY(14, 3, 4, 4, false)
#undef WT_TRY
#endif
  if (vec)
    return nw == 8 ? launch_wgrad<L, 8, true, WGeoRuntime>(a, pl, stream) : launch_wgrad<L, 4, true, WGeoRuntime>(a, pl, stream);
  return nw == 8 ? launch_wgrad<L, 8, false, WGeoRuntime>(a, pl, stream) : launch_wgrad<L, 4, false, WGeoRuntime>(a, pl, stream);
}

}  // namespace

Mfma2dWgradQuery mfma2d_wgrad_query(int B, int C, int H, int W, int K, int L, int dtype) {
  Mfma2dWgradQuery r = {false, 0, 0};
  if (mfma_mode() <= 0 || dtype != WTCONV_BF16 || K > 5 || L < 1 || L > kMaxLevels) return r;
  if (C > 65535) return r;
  const WVal& v = wplan_cached(B, C, H, W, L);
  if (!v.ok || v.nchunk > 65535) return r;
  r.ok = true;
  r.nchunk = v.nchunk;
  r.ws_bytes = static_cast<size_t>(v.nchunk) * C * ((1 + 4 * L) * K * K + 1) * sizeof(float);
  return r;
}

int mfma2d_wgrad_pass(const char* fn, const void* x, const void* grad_out, float* partial, int B, int C, int H, int W,
                      int K, int L, const FinishArgs& fin, hipStream_t stream) {
  const WVal& v = wplan_cached(B, C, H, W, L);
  if (!v.ok) return fail(WTCONV_E_UNSUPPORTED, "%s: shape not covered by the matrix-core kernels", fn);
  WPlan pl = v.pl;
  const bool aligned = ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(grad_out)) & 7u) == 0;
  const bool vec = (W % 4 == 0) && aligned;
  const WgradArgs a = {x, grad_out, partial, K, v.bchunk, v.nchunk, fin};
  switch (L) {
    case 1: return launch_wgrad_l<1>(v.nw, v.compact != 0, vec, a, pl, stream);
    case 2: return launch_wgrad_l<2>(v.nw, v.compact != 0, vec, a, pl, stream);
    case 3: return launch_wgrad_l<3>(v.nw, v.compact != 0, vec, a, pl, stream);
    case 4: return launch_wgrad_l<4>(v.nw, v.compact != 0, vec, a, pl, stream);
    default: return launch_wgrad_l<5>(v.nw, v.compact != 0, vec, a, pl, stream);
  }
}

}  // namespace wt
