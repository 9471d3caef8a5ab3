// Host-side planning: LDS layouts and launch geometry.  Pure C++, no device code.
#pragma once

#include <stddef.h>
#include <stdint.h>

#include "host_util.h"
#include "kernels1d.h"
#include "kernels2d.h"

namespace wt {

constexpr int round_up(int v, int m) { return (v + m - 1) / m * m; }

// Strip widths of the 2-D kernels (outputs per work item along a row).
constexpr int kTJC = 1;     // coarser levels of the plane kernel: single coefficients keep the most lanes busy
                            // (measured against strips of 2: 28x28 planes 106 -> 100 us, 14x14 73 -> 71, 56x56 equal)
constexpr int kTJW = 4;     // weight-gradient correlation strips

constexpr int pow2_ceil(int v) { int p = 1; while (p < v) p *= 2; return p; }
constexpr int log2_int(int v) { int s = 0; while ((1 << s) < v) ++s; return s; }

// Level-1 strip width and threads per plane of the plane kernel: the pair that keeps most
// lanes busy in the level-1 phase (ties: the wider strip, which reads less LDS per FMA),
// discounted when the slots of a workgroup (256 / threads-per-plane planes of
// `plane_lds_bytes` each) leave room for fewer than three workgroups per CU: with two, the
// phases of a plane are latency bound (measured on 14x14 planes: 88 -> 76 us with 32 instead
// of 16 threads per plane, i.e. half the slots).
constexpr void choose_plane_shape(int h1, int w1, size_t plane_lds_bytes, int* tj1, int* sg_shift) {
  double best = -1.0;
  for (int tj = 4; tj >= 1; tj /= 2) {
    const int gs = pow2_ceil((w1 + tj - 1) / tj);
    int sg = pow2_ceil(gs * h1);
    if (sg < 16) sg = 16;
    if (sg > 256) sg = 256;
    const int rpp = sg / gs > 0 ? sg / gs : 1;
    const int passes = (h1 + rpp - 1) / rpp;
    double eff = static_cast<double>(h1) * w1 / (static_cast<double>(sg) * passes * tj);
    const size_t wg_lds = plane_lds_bytes * (256 / sg);
    const int resident = wg_lds ? static_cast<int>(kLdsLimitBytes / wg_lds) : 3;
    if (resident < 3) eff *= (resident > 0 ? resident : 0.5) / 3.0;
    if (eff > best + 1e-9) { best = eff; *tj1 = tj; *sg_shift = log2_int(sg); }
  }
}

// Fills the LDS layout of one plane.  Planes are stacked in one column: x, then the four
// sub-band planes of level 1, level 2, ...; consecutive planes are separated by one gap of
// P zero rows that serves as bottom halo of the upper and top halo of the lower plane.
// with_grad_pyramid adds the padded pyramid of grad_out used by the weight-gradient kernel
// (and drops the Z buffers it does not need).
constexpr Plan2D make_plan2d_geometry(int B, int C, int H, int W, int K, int L, bool with_grad_pyramid, int nthreads,
                                      int pb) {
  Plan2D pl = {};
  pl.B = B; pl.C = C; pl.H = H; pl.W = W; pl.L = L;
  pl.nplanes = B * C;
  const int R = K / 2;
  pl.P = R > 1 ? R : 1;
  pl.h[0] = H; pl.w[0] = W;
  for (int l = 1; l <= L; ++l) { pl.h[l] = (pl.h[l - 1] + 1) / 2; pl.w[l] = (pl.w[l - 1] + 1) / 2; }
  // element (r, col) of sub-band s of level l sits at aoff[l] + s*apl[l] + (r+P)*astr[l] + col + P
  int off = 0;            // start of the zero gap above the next plane
  for (int l = 0; l <= L; ++l) {
    pl.astr[l] = round_up(pl.w[l] + 2 * pl.P, 4);
    pl.apl[l] = pb * (pl.h[l] + pl.P) * pl.astr[l];        // pb planes stacked, P shared zero rows between them
    if (l > 0) off += pl.P * (pl.astr[l - 1] - pl.astr[l]);   // the gap keeps the wider stride of the level above
    pl.aoff[l] = off;
    off += pl.apl[l] * (l == 0 ? 1 : 4);
  }
  off += pl.P * pl.astr[L];                                   // bottom halo of the last plane
  if (!with_grad_pyramid) {
    for (int l = 2; l <= L; ++l) {
      pl.zstr[l] = pl.w[l - 1];
      pl.zoff[l] = off;
      off += round_up(pl.zstr[l] * pl.h[l - 1], 4);
    }
  } else {
    for (int l = 0; l <= L; ++l) {
      pl.gstr[l] = round_up(pl.w[l] + 1, 4);
      pl.gpl[l] = pb * (pl.h[l] + pl.P) * pl.gstr[l];      // same row pitch as the x pyramid
      pl.goff[l] = off;
      off += pl.gpl[l] * (l == 0 ? 1 : 4);
    }
  }
  pl.plane_lds_floats = round_up(off + kLdsSlackFloats, 4);
  pl.sg_shift = log2_int(nthreads);
  pl.pb = pb;
  pl.slot_shift = log2_int(nthreads);
  pl.lds_floats = pl.plane_lds_floats;
  pl.groups_per_channel = 1;
  pl.vec_ok = W % 4 == 0;                         // (and aligned pointers: make_plan2d)
  return pl;
}

inline Plan2D make_plan2d(int B, int C, int H, int W, int K, int L, bool with_grad_pyramid, int nthreads,
                          size_t elem_size, const void* p0, const void* p1, const void* p2, int pb = 1) {
  Plan2D pl = make_plan2d_geometry(B, C, H, W, K, L, with_grad_pyramid, nthreads, pb);
  const uintptr_t mask = 4 * elem_size - 1;       // 4-element vectors: 16 B (fp32) / 8 B (bf16)
  auto aligned = [mask](const void* p) { return p == nullptr || (reinterpret_cast<uintptr_t>(p) & mask) == 0; };
  pl.vec_ok = (W % 4 == 0) && aligned(p0) && aligned(p1) && aligned(p2);
  return pl;
}

// Completes a plan for the plane kernel: threads per plane, slots per workgroup, prefetch.
constexpr void finish_plane_plan(Plan2D* pl, int tj1_sg_shift) {
  pl->sg_shift = tj1_sg_shift;
  const int sg = 1 << pl->sg_shift;
  pl->block = 256;   // (two whole planes per 512-thread workgroup measured slower: lockstep phases)
  const int slots = pl->block / sg;
  pl->lds_floats = pl->plane_lds_floats * slots;
  const int ppw = sg < kWave ? kWave / sg : 1;
  pl->groups_per_channel = (pl->B + ppw - 1) / ppw;
  pl->prefetch = 0;
  pl->fuse = 1;
  if (pl->vec_ok) {
    const int gs = pow2_ceil(pl->W / 4);       // 2x4 pieces per row pair, one lane each
    const int rows_per_pass = sg / gs;
    pl->prefetch = rows_per_pass >= 1 && (pl->h[1] + rows_per_pass - 1) / rows_per_pass <= kFetchPasses;
    if (pl->prefetch && sg == pl->block && gs <= 16 && pl->L >= 2) pl->fuse = pl->L >= 3 ? 3 : 2;
  }
}

// Geometry of the plane kernel's plan: the run-time plan of the launch, or a compile-time constant for a shape
// whose rows are whole aligned vectors (the launcher checks that the two agree before it picks the constant).
struct PlaneGeoRuntime {
  static constexpr bool kStatic = false;
  static constexpr Plan2D plan() { return Plan2D{}; }
};
constexpr Plan2D static_plane_plan(int H, int W, int K, int L, int* tj1_out) {
  Plan2D pl = make_plan2d_geometry(1, 1, H, W, K, L, false, 256, 1);
  int tj1 = 4, sg_shift = 8;
  choose_plane_shape(pl.h[1], pl.w[1], static_cast<size_t>(pl.plane_lds_floats) * 4, &tj1, &sg_shift);
  while (sg_shift < 8 && static_cast<size_t>(pl.plane_lds_floats) * 4 * (256 >> sg_shift) > kLdsLimitBytes / 2) ++sg_shift;
  finish_plane_plan(&pl, sg_shift);
  if (tj1_out != nullptr) *tj1_out = tj1;
  return pl;
}
template <int H, int W, int K, int L>
struct PlaneGeoStatic {
  static constexpr bool kStatic = true;
  static constexpr Plan2D plan() { return static_plane_plan(H, W, K, L, nullptr); }
  static constexpr int tj1() { int t = 4; static_plane_plan(H, W, K, L, &t); return t; }
  static constexpr int mode() {
    const Plan2D p = plan();
    return (p.prefetch && p.fuse >= 2) ? 3 : p.prefetch ? 0 : p.vec_ok ? 1 : 2;
  }
};
// Whether two plans describe the same LDS layout and work split (everything but batch and channels).
inline bool same_plane_geometry(const Plan2D& a, const Plan2D& b) {
  if (a.H != b.H || a.W != b.W || a.L != b.L || a.P != b.P || a.lds_floats != b.lds_floats || a.vec_ok != b.vec_ok ||
      a.prefetch != b.prefetch || a.sg_shift != b.sg_shift || a.plane_lds_floats != b.plane_lds_floats ||
      a.fuse != b.fuse || a.block != b.block)
    return false;
  for (int l = 0; l <= a.L; ++l)
    if (a.h[l] != b.h[l] || a.w[l] != b.w[l] || a.aoff[l] != b.aoff[l] || a.astr[l] != b.astr[l] ||
        a.apl[l] != b.apl[l] || a.zoff[l] != b.zoff[l] || a.zstr[l] != b.zstr[l])
      return false;
  return true;
}

// Planes per iteration of the weight-gradient kernel: as many (of one channel, consecutive
// batch items, stacked vertically) as fit the LDS budget of two workgroups per CU, up to 16.
// Small planes leave most of the 512 threads idle and pay the per-iteration barriers for
// little work when taken one at a time (measured, bf16: 28x28 230 -> 197 us, 14x14 193 -> 160 us,
// 7x7 148 -> 137 us); a 56x56 plane fills the budget by itself.
constexpr int wgrad_planes_per_iter(int B, int H, int W, int K, int L) {
  int pb = B < 16 ? B : 16;
  if (pb < 1) pb = 1;
  while (pb > 1) {
    const Plan2D t = make_plan2d_geometry(B, 1, H, W, K, L, true, 512, pb);
    if (static_cast<size_t>(t.plane_lds_floats) * 4 <= 80 * 1024) break;
    --pb;
  }
  return pb;
}

// Completes a plan for the weight-gradient kernel: threads per stacked plane, prefetch.
constexpr void finish_wgrad_plan(Plan2D* pl, int K) {
  // the final reduction reuses the LDS as [8 waves][sets * K * K + 1] floats, which is more
  // than the pyramids of a single tiny plane take
  const int red_floats = round_up(8 * (wgrad_sets(pl->L) * K * K + 1), 4);
  if (pl->lds_floats < red_floats) pl->lds_floats = red_floats;
  const int slots = pow2_ceil(pl->pb);
  pl->slot_shift = log2_int(512 / slots);
  const int nps = 512 / slots;
  pl->prefetch = 0;
  pl->fuse = 1;
  if (pl->vec_ok) {
    const int gs = pow2_ceil(pl->W / 4);
    pl->prefetch = nps / gs >= pl->h[1];       // one 2x4 piece per thread covers the plane
    if (pl->prefetch && pl->pb == 1 && gs <= 16 && pl->L >= 2) pl->fuse = pl->L >= 3 ? 3 : 2;
  }
}

// Weight-gradient plan of a shape as a compile-time constant: PB planes per iteration, rows of whole aligned vectors.
template <int H, int W, int K, int L, int PB>
struct WgradGeoStatic {
  static constexpr bool kStatic = true;
  static constexpr Plan2D plan() {
    Plan2D pl = make_plan2d_geometry(PB, 1, H, W, K, L, true, 512, PB);
    finish_wgrad_plan(&pl, K);
    return pl;
  }
};
inline bool same_wgrad_geometry(const Plan2D& a, const Plan2D& b) {
  if (a.H != b.H || a.W != b.W || a.L != b.L || a.P != b.P || a.lds_floats != b.lds_floats || a.vec_ok != b.vec_ok ||
      a.prefetch != b.prefetch || a.pb != b.pb || a.slot_shift != b.slot_shift || a.fuse != b.fuse ||
      a.plane_lds_floats != b.plane_lds_floats)
    return false;
  for (int l = 0; l <= a.L; ++l)
    if (a.h[l] != b.h[l] || a.w[l] != b.w[l] || a.aoff[l] != b.aoff[l] || a.astr[l] != b.astr[l] ||
        a.apl[l] != b.apl[l] || a.goff[l] != b.goff[l] || a.gstr[l] != b.gstr[l] || a.gpl[l] != b.gpl[l])
      return false;
  return true;
}

// ---- 1-D ------------------------------------------------------------------------------
constexpr int kTJ1D = 4;     // level coefficients per work item in the 1-D kernels
constexpr int kTile1D = 1024;

inline Plan1D make_plan1d(int C, int N, int K, int L, bool with_grad_pyramid, size_t elem_size,
                          const void* p0, const void* p1, const void* p2) {
  Plan1D pl = {};
  pl.C = C; pl.N = N; pl.L = L;
  const int R = K / 2;
  const int gran = 1 << L;
  int T = round_up(N, gran);
  if (T > kTile1D) T = kTile1D;          // kTile1D is a multiple of 2^L for every L <= 5
  pl.T = T;
  pl.ntiles = (N + T - 1) / T;
  int off = 0;
  for (int l = 0; l <= L; ++l) {
    pl.tl[l] = T >> l;
    pl.hal[l] = R << (L - l);
    pl.apl[l] = round_up(pl.tl[l] + 2 * pl.hal[l], 4);
    pl.aoff[l] = off;
    off += pl.apl[l] * (l == 0 ? 1 : 2);
  }
  if (!with_grad_pyramid) {
    for (int l = 2; l <= L; ++l) { pl.zoff[l] = off; off += round_up(pl.tl[l - 1], 4); }
  } else {
    for (int l = 0; l <= L; ++l) {
      pl.gpl[l] = round_up(pl.tl[l], kTJ1D) + kTJ1D;
      pl.goff[l] = off;
      off += pl.gpl[l] * (l == 0 ? 1 : 2);
    }
  }
  pl.lds_floats = round_up(off + kLdsSlackFloats, 4);
  const size_t row_bytes = static_cast<size_t>(N) * elem_size;
  auto aligned = [](const void* p) { return p == nullptr || (reinterpret_cast<uintptr_t>(p) & 15u) == 0; };
  pl.vec_ok = (row_bytes % 16 == 0) && aligned(p0) && aligned(p1) && aligned(p2);
  return pl;
}

// (row, tile) pairs per workgroup of the 1-D weight-gradient kernel.
inline void wgrad_chunks1d(int B, int C, int ntiles, int* per_chunk, int* nchunk) {
  const int total = B * ntiles;
  int want = (2048 + C - 1) / C;
  if (want < 1) want = 1;
  if (want > total) want = total;
  int pc = (total + want - 1) / want;
  if (pc < 1) pc = 1;
  *per_chunk = pc;
  *nchunk = (total + pc - 1) / pc;
}

// Workgroups of a persistent kernel: as many as can be resident at once.
inline int resident_workgroups(int ncu, size_t lds_bytes, int waves_per_wg, int max_waves_per_simd) {
  const int by_lds = lds_bytes ? static_cast<int>(kLdsLimitBytes / lds_bytes) : 8;
  const int by_waves = (4 * max_waves_per_simd) / waves_per_wg;
  int per_cu = by_lds < by_waves ? by_lds : by_waves;
  if (per_cu < 1) per_cu = 1;
  return ncu * per_cu;
}

}  // namespace wt
