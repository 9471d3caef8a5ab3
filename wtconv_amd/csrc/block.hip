// Host side of the block-epilogue kernels (kernels_block.h): argument checks, tile choice, launches.
// Allocates nothing, never synchronises.
#include <stdint.h>

#include <type_traits>

#include "common.h"
#include "host_util.h"
#include "kernels_block.h"

namespace wt {
namespace {

// Largest power-of-two pixel tile (8..64) whose [C][tp + 1] elements of `esz` bytes, plus the per-pixel statistics,
// stay within 48 KB of LDS (three workgroups per CU); false if even 8 pixels do not fit or the sizes overflow the
// indexing.
// `ntile` tiles per workgroup: one in the forward kernels, two in the backward ones (budget 64 KB there).
bool make_block_tile(int C, int HW, size_t esz, int ntile, BlockTile* out, size_t* lds_bytes) {
  BlockTile t = {};
  t.C = C; t.HW = HW;
  int tp = 64;
  // tiles (rounded up to 16 bytes), then floats: two sets of partial sums [256 / p][p], per-pixel statistics [4][p],
  // weight and bias [2][C]
  auto tile_bytes = [&](int p) { return (static_cast<size_t>(ntile) * C * (p + 1) * esz + 15) / 16 * 16; };
  auto bytes = [&](int p) { return tile_bytes(p) + (2 * kBlockThreads + 4 * p + 2 * static_cast<size_t>(C)) * sizeof(float); };
  const size_t budget = ntile == 1 ? 48 * 1024 : 64 * 1024;
  while (tp > 8 && bytes(tp) > budget) tp >>= 1;
  if (bytes(tp) > kLdsLimitBytes) return false;
  while (tp > 8 && tp / 2 >= HW) tp >>= 1;          // tiny images: no lanes without a pixel
  t.tp = tp;
  t.aux = static_cast<int>(tile_bytes(tp) / sizeof(float));
  t.tp_shift = 0;
  while ((1 << t.tp_shift) < tp) ++t.tp_shift;
  t.tiles = (HW + tp - 1) / tp;
  // reciprocal of C, exact for every dividend below tp * C (checked)
  const unsigned long long m = ((1ull << 32) + C - 1) / C;
  if (m >= (1ull << 32)) return false;
  t.mg_c = static_cast<unsigned>(m);
  for (int v = 0; v < tp * C; v += 1)
    if (static_cast<int>((static_cast<unsigned long long>(v) * t.mg_c) >> 32) != v / C) return false;
  *out = t;
  *lds_bytes = bytes(tp);
  return true;
}

struct TileKey {
  int C, HW, esz;      // esz: bytes of a tile element, negated for the two-tile plans of the backward kernels
  bool operator==(const TileKey& o) const { return C == o.C && HW == o.HW && esz == o.esz; }
};
struct TileKeyHash {
  size_t operator()(const TileKey& k) const {
    return (static_cast<size_t>(k.C) << 32) ^ (static_cast<size_t>(k.HW) << 4) ^ static_cast<size_t>(k.esz + 8);
  }
};
struct TileVal { bool ok; BlockTile t; size_t lds; int esz; };      // esz: bytes of a tile element

const TileVal& block_tile_cached(int C, int HW, int esz, int ntile = 1) {
  static thread_local std::unordered_map<TileKey, TileVal, TileKeyHash> cache;
  const TileKey key = {C, HW, ntile == 1 ? esz : -esz};
  auto it = cache.find(key);
  if (it == cache.end()) {
    if (cache.size() > 4096) cache.clear();
    TileVal v = {};
    v.ok = make_block_tile(C, HW, static_cast<size_t>(esz), ntile, &v.t, &v.lds);
    v.esz = esz;
    it = cache.emplace(key, v).first;
  }
  return it->second;
}

// Plan of the register-resident channel norm (channel_norm_reg_kernel): G pixel groups of four per tile so that a thread
// holds at most `np_max` channel pairs; the padding of the pixel-major LDS tile that spreads a wave's writes best over
// the banks.  false: too many channels for the registers of a workgroup (the LDS-tile kernel takes the call).
constexpr int kNormPairs = 6;
constexpr int kSumSlices = 32;        // slices of the two-stage column sum
constexpr int kSumTickets = 64;       // its ticket words (column blocks of 64: up to 4096 columns)

size_t block_record_floats(int B, int tiles, int C) { return (static_cast<size_t>(B) * tiles * 2 * C + 63) / 64 * 64; }

bool make_norm_tile(int C, int HW, size_t esz, NormTile* out, size_t* lds_bytes) {
  const int C2 = C / 2, pw = static_cast<int>(esz) / 2;           // dwords per channel pair
  int gshift = 5;
  while (gshift > 0 && (static_cast<long long>(C2) << gshift) > 256LL * kNormPairs) --gshift;
  if (gshift < 1) return false;
  while (gshift > 1 && (2 << gshift) >= HW) --gshift;             // tiny images: no tile of which half is outside
  const int cd = C2 * pw;
  NormTile t = {};
  auto bytes = [&](int gs, int pd) { return (static_cast<size_t>(4 << gs) * pd + 8 * (4 << gs) + 2 * static_cast<size_t>(C)) * sizeof(float); };
  while (gshift > 1 && bytes(gshift, cd + 32) > 64 * 1024) --gshift;
  if (bytes(gshift, cd + 32) > static_cast<size_t>(kLdsLimitBytes)) return false;
  const int G = 1 << gshift;
  int best_pad = 0, best = 1 << 30;
  for (int pad = 0; pad < 32; ++pad) {
    int cnt[64] = {0};
    int worst = 0;
    for (int l = 0; l < 64; ++l) {
      const int g = l & (G - 1), e = l >> gshift;
      for (int d = 0; d < pw; ++d) {
        const int bank = (4 * g * (cd + pad) + e * pw + d) & 63;
        if (++cnt[bank] > worst) worst = cnt[bank];
      }
    }
    if (worst < best) { best = worst; best_pad = pad; }
  }
  t.C = C; t.HW = HW; t.gshift = gshift;
  t.tiles = (HW + 4 * G - 1) / (4 * G);
  t.pd = cd + best_pad;
  t.aux = 4 * G * t.pd;
  const unsigned long long m = ((1ull << 32) + cd - 1) / cd;
  if (m >= (1ull << 32)) return false;
  t.mg_cd = static_cast<unsigned>(m);
  for (int v = 0; v < 4 * G * cd; ++v)
    if (static_cast<int>((static_cast<unsigned long long>(v) * t.mg_cd) >> 32) != v / cd) return false;
  *out = t;
  *lds_bytes = bytes(gshift, t.pd);
  return true;
}

struct NormVal { bool ok; NormTile t; size_t lds; };

const NormVal& norm_tile_cached(int C, int HW, int esz) {
  static thread_local std::unordered_map<TileKey, NormVal, TileKeyHash> cache;
  const TileKey key = {C, HW, esz};
  auto it = cache.find(key);
  if (it == cache.end()) {
    if (cache.size() > 4096) cache.clear();
    NormVal v = {};
    v.ok = make_norm_tile(C, HW, static_cast<size_t>(esz), &v.t, &v.lds);
    it = cache.emplace(key, v).first;
  }
  return it->second;
}

// float_tile: the caller can keep bf16 tensors as floats in LDS; taken where that still gives 64 pixels per tile.
int check_block_args(const char* fn, int B, int C, int HW, int dtype, int pdtype, const TileVal** tv,
                     bool float_tile = false, int ntile = 1) {
  if (B <= 0 || C <= 0 || HW <= 0) return fail(WTCONV_E_ARG, "%s: sizes must be positive (got B=%d C=%d HW=%d)", fn, B, C, HW);
  if (C % 2) return fail(WTCONV_E_UNSUPPORTED, "%s: the channel count must be even (got %d)", fn, C);
  if ((dtype != WTCONV_F32 && dtype != WTCONV_BF16) || (pdtype != WTCONV_F32 && pdtype != WTCONV_BF16))
    return fail(WTCONV_E_ARG, "%s: unknown dtype code", fn);
  if (B > 65535) return fail(WTCONV_E_UNSUPPORTED, "%s: batch %d exceeds the launch grid", fn, B);
  if (static_cast<long long>(C) * HW > 0x7fffffffLL) return fail(WTCONV_E_UNSUPPORTED, "%s: an image of %d x %d elements is too large", fn, C, HW);
  const TileVal* vp = &block_tile_cached(C, HW, dtype == WTCONV_F32 ? 4 : 2, ntile);
  if (ntile == 1 && float_tile && dtype != WTCONV_F32) {
    const TileVal& vf = block_tile_cached(C, HW, 4);
    if (vf.ok && vf.t.tp == 64) vp = &vf;
  }
  const TileVal& v = *vp;
  if (!v.ok) return fail(WTCONV_E_UNSUPPORTED, "%s: %d channels do not fit a tile in LDS", fn, C);
  *tv = &v;
  return 0;
}

}  // namespace
}  // namespace wt

using namespace wt;

extern "C" int wtconv_channel_norm(const void* x, void* out, const void* weight, const void* bias, int B, int C, int HW,
                                   float eps, int dtype, int param_dtype, int out_nhwc, void* stream_) {
  const char* fn = "wtconv_channel_norm";
  const TileVal* tv = nullptr;
  if (int e = check_block_args(fn, B, C, HW, dtype, param_dtype, &tv, true)) return e;
  if (x == nullptr || out == nullptr || weight == nullptr || bias == nullptr) return fail(WTCONV_E_ARG, "%s: null pointer", fn);
  if (x == out) return fail(WTCONV_E_ARG, "%s: in-place use is not supported (tiles of the output overlap other tiles' input)", fn);
  const size_t esz = dtype == WTCONV_F32 ? 4 : 2;
  if ((reinterpret_cast<uintptr_t>(x) % esz) || (reinterpret_cast<uintptr_t>(out) % (2 * esz)))
    return fail(WTCONV_E_ARG, "%s: tensor pointer not aligned (input to one element, output to two)", fn);
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  const dim3 grid(tv->t.tiles, B);
  // rows of whole aligned 4-element vectors move as such
  const bool vec = HW % 4 == 0 && reinterpret_cast<uintptr_t>(x) % (4 * esz) == 0;
  // every value of a tile in a register of its own, where the channels fit
  {
    // (rows that move element by element: measured no faster than the LDS-tile kernel below, which keeps them)
    const bool v4 = vec && (out_nhwc || reinterpret_cast<uintptr_t>(out) % (4 * esz) == 0);
    const NormVal& nv = norm_tile_cached(C, HW, static_cast<int>(esz));
    if (nv.ok && v4) {
      auto launch_reg = [&](auto kern, auto* tag) {
        using T = std::remove_pointer_t<decltype(tag)>;
        if (int e = allow_lds(kern, nv.lds)) return e;
        WT_LAUNCH(kern, dim3(nv.t.tiles, B), dim3(kBlockThreads), nv.lds, stream, static_cast<const T*>(x),
                  static_cast<T*>(out), weight, bias, param_dtype, eps, nv.t);
        return check_launch("channel_norm_reg_kernel");
      };
      auto by_layout = [&](auto* tag) {
        using T = std::remove_pointer_t<decltype(tag)>;
        if (v4) return out_nhwc ? launch_reg(channel_norm_reg_kernel<T, kNormPairs, true, true>, tag)
                                : launch_reg(channel_norm_reg_kernel<T, kNormPairs, false, true>, tag);
        return out_nhwc ? launch_reg(channel_norm_reg_kernel<T, kNormPairs, true, false>, tag)
                        : launch_reg(channel_norm_reg_kernel<T, kNormPairs, false, false>, tag);
      };
      return dtype == WTCONV_F32 ? by_layout(static_cast<float*>(nullptr)) : by_layout(static_cast<bf16_t*>(nullptr));
    }
  }
  auto launch = [&](auto kern, auto* tag) {
    using T = std::remove_pointer_t<decltype(tag)>;
    if (int e = allow_lds(kern, tv->lds)) return e;
    WT_LAUNCH(kern, grid, dim3(kBlockThreads), tv->lds, stream, static_cast<const T*>(x), static_cast<T*>(out),
              weight, bias, param_dtype, eps, out_nhwc, tv->t);
    return check_launch("channel_norm_kernel");
  };
  if (dtype == WTCONV_F32)
    return vec ? launch(channel_norm_kernel<float, float, true>, static_cast<float*>(nullptr))
               : launch(channel_norm_kernel<float, float, false>, static_cast<float*>(nullptr));
  if (tv->esz == 4)      // bf16 tensor, tile of floats
    return vec ? launch(channel_norm_kernel<bf16_t, float, true>, static_cast<bf16_t*>(nullptr))
               : launch(channel_norm_kernel<bf16_t, float, false>, static_cast<bf16_t*>(nullptr));
  return vec ? launch(channel_norm_kernel<bf16_t, bf16_t, true>, static_cast<bf16_t*>(nullptr))
             : launch(channel_norm_kernel<bf16_t, bf16_t, false>, static_cast<bf16_t*>(nullptr));
}

extern "C" int wtconv_block_residual(const void* y, const void* shortcut, const void* gamma, void* out, int B, int C,
                                     int HW, int dtype, int param_dtype, void* stream_) {
  const char* fn = "wtconv_block_residual";
  const TileVal* tv = nullptr;
  if (int e = check_block_args(fn, B, C, HW, dtype, param_dtype, &tv)) return e;
  if (y == nullptr || shortcut == nullptr || out == nullptr) return fail(WTCONV_E_ARG, "%s: null pointer", fn);
  if (y == out) return fail(WTCONV_E_ARG, "%s: the output may alias the shortcut, not the NHWC input", fn);
  const size_t esz = dtype == WTCONV_F32 ? 4 : 2;
  if ((reinterpret_cast<uintptr_t>(y) % (2 * esz)) || (reinterpret_cast<uintptr_t>(shortcut) % esz) ||
      (reinterpret_cast<uintptr_t>(out) % esz))
    return fail(WTCONV_E_ARG, "%s: tensor pointer not aligned (NHWC input to two elements, the others to one)", fn);
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  const dim3 grid(tv->t.tiles, B);
  const bool vec = HW % 4 == 0 && reinterpret_cast<uintptr_t>(shortcut) % (4 * esz) == 0 &&
                   reinterpret_cast<uintptr_t>(out) % (4 * esz) == 0;
  {
    const NormVal& nv = norm_tile_cached(C, HW, static_cast<int>(esz));
    if (nv.ok && vec) {      // (element-wise rows: the LDS-tile kernel below measured faster)
      auto launch_reg = [&](auto kern, auto* tag) {
        using T = std::remove_pointer_t<decltype(tag)>;
        if (int e = allow_lds(kern, nv.lds)) return e;
        WT_LAUNCH(kern, dim3(nv.t.tiles, B), dim3(kBlockThreads), nv.lds, stream, static_cast<const T*>(y),
                  static_cast<const T*>(shortcut), gamma, param_dtype, static_cast<T*>(out), nv.t);
        return check_launch("block_residual_reg_kernel");
      };
      auto by_rows = [&](auto* tag) {
        using T = std::remove_pointer_t<decltype(tag)>;
        return vec ? launch_reg(block_residual_reg_kernel<T, kNormPairs, true>, tag)
                   : launch_reg(block_residual_reg_kernel<T, kNormPairs, false>, tag);
      };
      return dtype == WTCONV_F32 ? by_rows(static_cast<float*>(nullptr)) : by_rows(static_cast<bf16_t*>(nullptr));
    }
  }
  auto launch = [&](auto kern, auto* tag) {
    using T = std::remove_pointer_t<decltype(tag)>;
    if (int e = allow_lds(kern, tv->lds)) return e;
    WT_LAUNCH(kern, grid, dim3(kBlockThreads), tv->lds, stream, static_cast<const T*>(y), static_cast<const T*>(shortcut),
              gamma, param_dtype, static_cast<T*>(out), tv->t);
    return check_launch("block_residual_kernel");
  };
  if (dtype == WTCONV_F32)
    return vec ? launch(block_residual_kernel<float, true>, static_cast<float*>(nullptr))
               : launch(block_residual_kernel<float, false>, static_cast<float*>(nullptr));
  return vec ? launch(block_residual_kernel<bf16_t, true>, static_cast<bf16_t*>(nullptr))
             : launch(block_residual_kernel<bf16_t, false>, static_cast<bf16_t*>(nullptr));
}

// ---- backward passes ---------------------------------------------------------------------------------------

// Floats of workspace: one record per workgroup (B * tiles of them) of 2 C floats (the norm's dweight and dbias; the
// residual's dgamma takes the first C of each).
extern "C" size_t wtconv_block_workspace_bytes(int B, int C, int HW, int dtype) {
  if (B <= 0 || C <= 0 || HW <= 0 || (dtype != WTCONV_F32 && dtype != WTCONV_BF16)) return 0;
  const TileVal& v = block_tile_cached(C, HW, dtype == WTCONV_F32 ? 4 : 2, 2);
  if (!v.ok) return 0;
  int tiles = v.t.tiles;                       // whichever plan a call takes: the larger record count
  const NormVal& nv = norm_tile_cached(C, HW, dtype == WTCONV_F32 ? 4 : 2);
  if (nv.ok && nv.t.tiles > tiles) tiles = nv.t.tiles;
  // the records, then the slice sums and tickets of the two-stage column sum
  const size_t bytes = (block_record_floats(B, tiles, C) + static_cast<size_t>(kSumSlices) * 2 * C) * sizeof(float) +
                       kSumTickets * sizeof(unsigned);
  return (bytes + 255) / 256 * 256;
}

// Two-stage column sum of the register-plan kernels: slice sums and tickets behind the records (`rec_floats` of them;
// the kernel that wrote the records has cleared the tickets).
static unsigned* sum_tickets(float* partial, size_t rec_floats, int C) {
  return reinterpret_cast<unsigned*>(partial + rec_floats + static_cast<size_t>(kSumSlices) * 2 * C);
}

static int launch_column_sum_sliced(float* partial, size_t rec_floats, int C, int nrec, int ncol, float* out0,
                                    float* out1, int split, hipStream_t stream) {
  int ns = nrec / 16;                          // at least 16 records per slice
  if (ns > kSumSlices) ns = kSumSlices;
  if (ns < 1) ns = 1;
  WT_LAUNCH(column_sum_sliced_kernel, dim3((ncol + 63) / 64, ns), dim3(kBlockThreads), 0, stream, partial, nrec, ncol,
            partial + rec_floats, sum_tickets(partial, rec_floats, C), out0, out1, split);
  return check_launch("column_sum_sliced_kernel");
}

static int launch_column_sum(const float* partial, int nrec, int ncol, float* out0, float* out1, int split,
                             hipStream_t stream) {
  WT_LAUNCH(column_sum_kernel, dim3((ncol + 63) / 64), dim3(kBlockThreads), 0, stream, partial, nrec, ncol, out0, out1,
            split);
  return check_launch("column_sum_kernel");
}

extern "C" int wtconv_channel_norm_backward(const void* x, const void* dy, const void* weight, void* dx, float* dweight,
                                            float* dbias, int B, int C, int HW, float eps, int dtype, int param_dtype,
                                            int dy_nhwc, void* workspace, size_t workspace_bytes, void* stream_) {
  const char* fn = "wtconv_channel_norm_backward";
  const TileVal* tv = nullptr;
  if (int e = check_block_args(fn, B, C, HW, dtype, param_dtype, &tv, false, 2)) return e;
  if (x == nullptr || dy == nullptr || weight == nullptr || dx == nullptr || dweight == nullptr || dbias == nullptr)
    return fail(WTCONV_E_ARG, "%s: null pointer", fn);
  const size_t esz = dtype == WTCONV_F32 ? 4 : 2;
  if ((reinterpret_cast<uintptr_t>(x) % esz) || (reinterpret_cast<uintptr_t>(dx) % (2 * esz)) ||
      (reinterpret_cast<uintptr_t>(dy) % (2 * esz)))
    return fail(WTCONV_E_ARG, "%s: tensor pointer not aligned (x to one element, dy and dx to two)", fn);
  const size_t need = wtconv_block_workspace_bytes(B, C, HW, dtype);
  if (workspace == nullptr || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) % 4))
    return fail(WTCONV_E_WORKSPACE, "%s: workspace of %zu B needed, %zu given", fn, need, workspace_bytes);
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  const dim3 grid(tv->t.tiles, B);
  const bool vec = HW % 4 == 0 && reinterpret_cast<uintptr_t>(x) % (4 * esz) == 0 &&
                   reinterpret_cast<uintptr_t>(dx) % (4 * esz) == 0 &&
                   (dy_nhwc || reinterpret_cast<uintptr_t>(dy) % (4 * esz) == 0);
  float* partial = static_cast<float*>(workspace);
  {
    const NormVal& nv = norm_tile_cached(C, HW, static_cast<int>(esz));
    const size_t lds = nv.ok ? (static_cast<size_t>(nv.t.aux) + 16 * (4 << nv.t.gshift) + C) * sizeof(float) : 0;
    if (nv.ok && lds <= 64 * 1024 && 2 * C <= 64 * kSumTickets) {
      const size_t rec_floats = block_record_floats(B, nv.t.tiles, C);
      auto launch_reg = [&](auto kern, auto* tag) {
        using T = std::remove_pointer_t<decltype(tag)>;
        if (int e = allow_lds(kern, lds)) return e;
        WT_LAUNCH(kern, dim3(nv.t.tiles, B), dim3(kBlockThreads), lds, stream, static_cast<const T*>(x),
                  static_cast<const T*>(dy), weight, param_dtype, eps, static_cast<T*>(dx), partial, nv.t,
                  sum_tickets(partial, rec_floats, C), kSumTickets);
        return check_launch("channel_norm_bwd_reg_kernel");
      };
      auto by_layout = [&](auto* tag) {
        using T = std::remove_pointer_t<decltype(tag)>;
        if (vec) return dy_nhwc ? launch_reg(channel_norm_bwd_reg_kernel<T, kNormPairs, true, true>, tag)
                                : launch_reg(channel_norm_bwd_reg_kernel<T, kNormPairs, false, true>, tag);
        return dy_nhwc ? launch_reg(channel_norm_bwd_reg_kernel<T, kNormPairs, true, false>, tag)
                       : launch_reg(channel_norm_bwd_reg_kernel<T, kNormPairs, false, false>, tag);
      };
      const int e = dtype == WTCONV_F32 ? by_layout(static_cast<float*>(nullptr)) : by_layout(static_cast<bf16_t*>(nullptr));
      if (e) return e;
      return launch_column_sum_sliced(partial, rec_floats, C, B * nv.t.tiles, 2 * C, dweight, dbias, C, stream);
    }
  }
  auto launch = [&](auto kern, auto* tag) {
    using T = std::remove_pointer_t<decltype(tag)>;
    if (int e = allow_lds(kern, tv->lds)) return e;
    WT_LAUNCH(kern, grid, dim3(kBlockThreads), tv->lds, stream, static_cast<const T*>(x), static_cast<const T*>(dy),
              weight, param_dtype, eps, dy_nhwc, static_cast<T*>(dx), partial, tv->t);
    return check_launch("channel_norm_bwd_kernel");
  };
  int e;
  if (dtype == WTCONV_F32)
    e = vec ? launch(channel_norm_bwd_kernel<float, true>, static_cast<float*>(nullptr))
            : launch(channel_norm_bwd_kernel<float, false>, static_cast<float*>(nullptr));
  else
    e = vec ? launch(channel_norm_bwd_kernel<bf16_t, true>, static_cast<bf16_t*>(nullptr))
            : launch(channel_norm_bwd_kernel<bf16_t, false>, static_cast<bf16_t*>(nullptr));
  if (e) return e;
  return launch_column_sum(partial, B * tv->t.tiles, 2 * C, dweight, dbias, C, stream);
}

extern "C" int wtconv_block_residual_backward(const void* dout, const void* y, const void* gamma, void* dy, float* dgamma,
                                              int B, int C, int HW, int dtype, int param_dtype, void* workspace,
                                              size_t workspace_bytes, void* stream_) {
  const char* fn = "wtconv_block_residual_backward";
  const TileVal* tv = nullptr;
  if (int e = check_block_args(fn, B, C, HW, dtype, param_dtype, &tv, false, 2)) return e;
  if (dout == nullptr || y == nullptr || gamma == nullptr || dy == nullptr || dgamma == nullptr)
    return fail(WTCONV_E_ARG, "%s: null pointer", fn);
  const size_t esz = dtype == WTCONV_F32 ? 4 : 2;
  if ((reinterpret_cast<uintptr_t>(dout) % esz) || (reinterpret_cast<uintptr_t>(y) % (2 * esz)) ||
      (reinterpret_cast<uintptr_t>(dy) % (2 * esz)))
    return fail(WTCONV_E_ARG, "%s: tensor pointer not aligned (dout to one element, the NHWC tensors to two)", fn);
  const size_t need = wtconv_block_workspace_bytes(B, C, HW, dtype);
  if (workspace == nullptr || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) % 4))
    return fail(WTCONV_E_WORKSPACE, "%s: workspace of %zu B needed, %zu given", fn, need, workspace_bytes);
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  const dim3 grid(tv->t.tiles, B);
  const bool vec = HW % 4 == 0 && reinterpret_cast<uintptr_t>(dout) % (4 * esz) == 0;
  float* partial = static_cast<float*>(workspace);
  {
    const NormVal& nv = norm_tile_cached(C, HW, static_cast<int>(esz));
    if (nv.ok && C <= 64 * kSumTickets) {
      const size_t rec_floats = block_record_floats(B, nv.t.tiles, C);
      auto launch_reg = [&](auto kern, auto* tag) {
        using T = std::remove_pointer_t<decltype(tag)>;
        if (int e = allow_lds(kern, nv.lds)) return e;
        WT_LAUNCH(kern, dim3(nv.t.tiles, B), dim3(kBlockThreads), nv.lds, stream, static_cast<const T*>(dout),
                  static_cast<const T*>(y), gamma, param_dtype, static_cast<T*>(dy), partial, nv.t,
                  sum_tickets(partial, rec_floats, C), kSumTickets);
        return check_launch("block_residual_bwd_reg_kernel");
      };
      auto by_rows = [&](auto* tag) {
        using T = std::remove_pointer_t<decltype(tag)>;
        return vec ? launch_reg(block_residual_bwd_reg_kernel<T, kNormPairs, true>, tag)
                   : launch_reg(block_residual_bwd_reg_kernel<T, kNormPairs, false>, tag);
      };
      const int e = dtype == WTCONV_F32 ? by_rows(static_cast<float*>(nullptr)) : by_rows(static_cast<bf16_t*>(nullptr));
      if (e) return e;
      return launch_column_sum_sliced(partial, rec_floats, C, B * nv.t.tiles, C, dgamma, dgamma, C, stream);
    }
  }
  auto launch = [&](auto kern, auto* tag) {
    using T = std::remove_pointer_t<decltype(tag)>;
    if (int e = allow_lds(kern, tv->lds)) return e;
    WT_LAUNCH(kern, grid, dim3(kBlockThreads), tv->lds, stream, static_cast<const T*>(dout), static_cast<const T*>(y),
              gamma, param_dtype, static_cast<T*>(dy), partial, tv->t);
    return check_launch("block_residual_bwd_kernel");
  };
  int e;
  if (dtype == WTCONV_F32)
    e = vec ? launch(block_residual_bwd_kernel<float, true>, static_cast<float*>(nullptr))
            : launch(block_residual_bwd_kernel<float, false>, static_cast<float*>(nullptr));
  else
    e = vec ? launch(block_residual_bwd_kernel<bf16_t, true>, static_cast<bf16_t*>(nullptr))
            : launch(block_residual_bwd_kernel<bf16_t, false>, static_cast<bf16_t*>(nullptr));
  if (e) return e;
  return launch_column_sum(partial, B * tv->t.tiles, C, dgamma, dgamma, C, stream);
}
