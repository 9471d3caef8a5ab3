// What a WTConvNeXt block does around its WTConv layer (wtconvnext/wtconvnext.py:125-140 of the reference): after
// `conv_dw` the activations are permuted to NHWC and LayerNorm-ed over the channels (:132-133); after the MLP they
// are permuted back, scaled per channel and added to the shortcut (:135-140).  As separate passes these are four
// trips through HBM, two of them layout copies; here each side is one kernel that transposes through LDS:
//   channel_norm_kernel    NCHW -> LayerNorm over C -> NHWC (or NCHW: the LayerNorm2d of stem and downsample layers)
//   block_residual_kernel  NHWC y, NCHW shortcut -> shortcut + gamma[c] * y, NCHW
// A workgroup takes a tile of TP consecutive pixels of one image with all their channels: [C][TP + 1] elements in
// LDS, in the tensors' own element type (the values pass through unchanged; bf16 tiles are half the size, so twice
// the pixels fit: longer contiguous runs on the NCHW side and more workgroups per CU).  The odd row pitch keeps
// both the pixel-major and the channel-major sweep free of bank conflicts.  The NCHW side moves TP contiguous
// elements per channel, the NHWC side the tile's TP * C elements, which are one contiguous run.  Statistics are
// two sweeps over LDS in fp32 (mean, then the sum of squared deviations).
#pragma once

#include <type_traits>

#include "common.h"

namespace wt {

constexpr int kBlockThreads = 256;

struct BlockTile {
  int C, HW;
  int tp;            // pixels per tile: a power of two, 8..128
  int aux;           // float index in LDS where the arrays behind the tile start
  int tp_shift;
  int tiles;         // tiles per image
  unsigned mg_c;     // reciprocal of C for dividends < tp * C (shift 32)
};

__device__ __forceinline__ int div_c(int v, unsigned magic) {
#ifdef WT_EMULATE
  return static_cast<int>((static_cast<unsigned long long>(static_cast<unsigned>(v)) * magic) >> 32);
#else
  return static_cast<int>(__umulhi(static_cast<unsigned>(v), magic));
#endif
}

// The (tile, image) of a workgroup of a (tiles, B) grid, dealt so that the workgroups of one XCD hold consecutive tiles
// (xcd_contiguous): where a tile's rows are shorter than a cache line, neighbouring tiles share lines, which then meet
// in one L2.
__device__ __forceinline__ void tile_of_workgroup(int& tile, int& b) {
  const int tiles = static_cast<int>(gridDim.x);
  const int i = xcd_contiguous(static_cast<int>(blockIdx.x) + tiles * static_cast<int>(blockIdx.y), tiles * static_cast<int>(gridDim.y));
  b = i / tiles;
  tile = i - b * tiles;
}

template <typename T>
__device__ __forceinline__ void store_pair(T* p, float a, float b);
template <> __device__ __forceinline__ void store_pair<float>(float* p, float a, float b) {
  float2 v;
  v.x = a; v.y = b;
  *reinterpret_cast<float2*>(p) = v;
}
template <> __device__ __forceinline__ void store_pair<bf16_t>(bf16_t* p, float a, float b) {
  *reinterpret_cast<uint32_t*>(p) = pack_bf16x2(a, b);
}
// two consecutive elements as they are
template <typename T>
__device__ __forceinline__ void load_pair_raw(const T* p, T& a, T& b);
template <> __device__ __forceinline__ void load_pair_raw<float>(const float* p, float& a, float& b) {
  const float2 v = *reinterpret_cast<const float2*>(p);
  a = v.x; b = v.y;
}
template <> __device__ __forceinline__ void load_pair_raw<bf16_t>(const bf16_t* p, bf16_t& a, bf16_t& b) {
  const uint32_t v = *reinterpret_cast<const uint32_t*>(p);
  a = static_cast<bf16_t>(v); b = static_cast<bf16_t>(v >> 16);
}
template <typename T>
__device__ __forceinline__ void load_pair(const T* p, float& a, float& b);
template <> __device__ __forceinline__ void load_pair<float>(const float* p, float& a, float& b) {
  const float2 v = *reinterpret_cast<const float2*>(p);
  a = v.x; b = v.y;
}
template <> __device__ __forceinline__ void load_pair<bf16_t>(const bf16_t* p, float& a, float& b) {
  const uint32_t v = *reinterpret_cast<const uint32_t*>(p);
  a = __uint_as_float(v << 16); b = __uint_as_float(v & 0xffff0000u);
}

// four consecutive elements at an address aligned to four elements
template <typename T> struct Quad;
template <> struct Quad<float> {
  float4 v;
  __device__ __forceinline__ void load(const float* p) { v = *reinterpret_cast<const float4*>(p); }
  // the first n of four elements one by one (any alignment), the rest zero
  __device__ __forceinline__ void load_n(const float* p, int n) {
    v.x = n > 0 ? p[0] : 0.f; v.y = n > 1 ? p[1] : 0.f; v.z = n > 2 ? p[2] : 0.f; v.w = n > 3 ? p[3] : 0.f;
  }
  __device__ __forceinline__ void get(float (&f)[4]) const { f[0] = v.x; f[1] = v.y; f[2] = v.z; f[3] = v.w; }
  __device__ __forceinline__ void raw(float (&f)[4]) const { get(f); }
};
template <> struct Quad<bf16_t> {
  uint2 v;
  __device__ __forceinline__ void load(const bf16_t* p) { v = *reinterpret_cast<const uint2*>(p); }
  __device__ __forceinline__ void load_n(const bf16_t* p, int n) {
    const uint32_t a = n > 0 ? p[0] : 0u, b = n > 1 ? p[1] : 0u, c = n > 2 ? p[2] : 0u, d = n > 3 ? p[3] : 0u;
    v.x = a | (b << 16); v.y = c | (d << 16);
  }
  __device__ __forceinline__ void get(float (&f)[4]) const {
    f[0] = __uint_as_float(v.x << 16); f[1] = __uint_as_float(v.x & 0xffff0000u);
    f[2] = __uint_as_float(v.y << 16); f[3] = __uint_as_float(v.y & 0xffff0000u);
  }
  __device__ __forceinline__ void raw(bf16_t (&f)[4]) const {
    f[0] = static_cast<bf16_t>(v.x); f[1] = static_cast<bf16_t>(v.x >> 16);
    f[2] = static_cast<bf16_t>(v.y); f[3] = static_cast<bf16_t>(v.y >> 16);
  }
};

constexpr int kQuadBatch = 6;      // vector loads a thread keeps in flight before it writes them to LDS

// tile element from / to fp32 (LT = float or the tensor's type)
template <typename LT> __device__ __forceinline__ float tile_get(LT v) { return to_f32<LT>(v); }

// NCHW tile -> LDS [C][tp + 1] of LT (float, or T itself); pixels past the image are left alone (never read back).
// VEC: HW is a multiple of 4 and the tensor 4-element aligned, so rows move as 4-element vectors.
template <typename T, typename LT, bool VEC>
__device__ __forceinline__ void tile_from_nchw(const T* __restrict__ img, LT* lds, const BlockTile& t, int p0, int tid) {
  const int pitch = t.tp + 1;
  if constexpr (VEC) {
    const int gshift = t.tp_shift - 2;                       // 4-pixel groups per tile row
    const int g = tid & ((1 << gshift) - 1), c0 = tid >> gshift, cstep = kBlockThreads >> gshift;
    const int p = 4 * g;
    if (p0 + p < t.HW) {                                     // (HW % 4 == 0: a group is inside the image or outside)
      const T* src = img + p0 + p;
      for (int cb = c0; cb < t.C; cb += kQuadBatch * cstep) {
        Quad<T> q[kQuadBatch];
#pragma unroll
        for (int k = 0; k < kQuadBatch; ++k) {
          const int c = cb + k * cstep;
          if (c < t.C) q[k].load(src + static_cast<size_t>(c) * t.HW);
        }
#pragma unroll
        for (int k = 0; k < kQuadBatch; ++k) {
          const int c = cb + k * cstep;
          if (c < t.C) {
            LT f[4];
            if constexpr (std::is_same<LT, T>::value) q[k].raw(f);
            else q[k].get(f);
#pragma unroll
            for (int j = 0; j < 4; ++j) lds[c * pitch + p + j] = f[j];
          }
        }
      }
    }
  } else {
    const int p = tid & (t.tp - 1), c0 = tid >> t.tp_shift, cstep = kBlockThreads >> t.tp_shift;
    if (p0 + p < t.HW)
      for (int c = c0; c < t.C; c += cstep) {
        const T v = img[static_cast<size_t>(c) * t.HW + p0 + p];
        if constexpr (std::is_same<LT, T>::value) lds[c * pitch + p] = v;
        else lds[c * pitch + p] = to_f32<T>(v);
      }
  }
}

// Grid (tiles, B).  out_nhwc != 0: out is (B, HW, C); else (B, C, HW).  LT: the tile's element type -- fp32 where
// that reaches 64 pixels per tile (the three sweeps over the tile then cost no conversions), else T.
template <typename T, typename LT, bool VEC>
__global__ void __launch_bounds__(kBlockThreads)
channel_norm_kernel(const T* __restrict__ x, T* __restrict__ out, const void* __restrict__ weight,
                    const void* __restrict__ bias, int pdtype, float eps, int out_nhwc, const BlockTile t) {
  WT_SHARED_FLOATS(ldsf);
  LT* lds = reinterpret_cast<LT*>(ldsf);         // the tile
  const int tid = threadIdx.x;
  int tile, b;
  tile_of_workgroup(tile, b);
  const int p0 = tile * t.tp;
  const int pitch = t.tp + 1, C = t.C;
  const int np = t.HW - p0 < t.tp ? t.HW - p0 : t.tp;
  float* psum = ldsf + t.aux;                    // [parts][tp] partial sums
  float* pvar = psum + kBlockThreads;            // [parts][tp] partial sums of squared deviations
  float* stat = pvar + kBlockThreads;            // mean[tp], rstd[tp]
  float* wgt = stat + 2 * t.tp;                  // weight[C], bias[C]
  const T* img = x + static_cast<size_t>(b) * C * t.HW;
  tile_from_nchw<T, LT, VEC>(img, lds, t, p0, tid);
  for (int c = tid; c < C; c += kBlockThreads) {
    wgt[c] = load_param(weight, pdtype, c);
    wgt[C + c] = load_param(bias, pdtype, c);
  }
  __syncthreads();
  const int p = tid & (t.tp - 1), part_i = tid >> t.tp_shift, parts = kBlockThreads >> t.tp_shift;
  const bool live = p < np;
  float s = 0.f;
  if (live)
    for (int c = part_i; c < C; c += parts) s += tile_get<LT>(lds[c * pitch + p]);
  psum[part_i * t.tp + p] = s;
  __syncthreads();
  float mean = 0.f;
  for (int k = 0; k < parts; ++k) mean += psum[k * t.tp + p];
  mean *= 1.f / static_cast<float>(C);
  float v = 0.f;
  if (live)
    for (int c = part_i; c < C; c += parts) {
      const float d = tile_get<LT>(lds[c * pitch + p]) - mean;
      v += d * d;
    }
  pvar[part_i * t.tp + p] = v;
  __syncthreads();
  float var = 0.f;
  for (int k = 0; k < parts; ++k) var += pvar[k * t.tp + p];
  const float rstd = 1.f / sqrtf(var * (1.f / static_cast<float>(C)) + eps);
  if (out_nhwc) {
    if (part_i == 0) { stat[p] = mean; stat[t.tp + p] = rstd; }
    __syncthreads();
    // the tile's output is one contiguous run of np * C elements; C is even, so pairs never straddle a pixel
    T* dst = out + (static_cast<size_t>(b) * t.HW + p0) * C;
    const int npair = (np * C) >> 1;
    for (int i = tid; i < npair; i += kBlockThreads) {
      const int e = 2 * i;
      const int pp = div_c(e, t.mg_c), c = e - pp * C;
      const float m = stat[pp], r = stat[t.tp + pp];
      const float a = (tile_get<LT>(lds[c * pitch + pp]) - m) * r * wgt[c] + wgt[C + c];
      const float bb = (tile_get<LT>(lds[(c + 1) * pitch + pp]) - m) * r * wgt[c + 1] + wgt[C + c + 1];
      store_pair<T>(dst + e, a, bb);
    }
  } else {
    T* dst = out + static_cast<size_t>(b) * C * t.HW + p0;
    if (live)
      for (int c = part_i; c < C; c += parts)
        dst[static_cast<size_t>(c) * t.HW + p] = from_f32<T>((tile_get<LT>(lds[c * pitch + p]) - mean) * rstd * wgt[c] + wgt[C + c]);
  }
}

// ---- channel norm with the tile's values held in registers -----------------------------------------------------
// Rows move as 4-element vectors (VEC: HW a multiple of 4, aligned tensors) or element by element.  A workgroup takes `tp` = 4 G consecutive pixels (G a power of two,
// 2..32) of one image; thread (g, e) = (tid % G, tid / G) owns pixels 4g..4g+3 of the channel pairs e, e + cs,
// e + 2 cs, ... (cs = 256 / G, at most NP pairs): every value of the tile sits in one register of one thread from its
// load to its store, the statistics are two exact passes over registers (mean, then squared deviations; partial sums
// meet across the lanes of a wave that share g, then across the four waves through LDS), and LDS carries each
// normalised value once, as the transpose to NHWC: a pixel-major tile [tp][pd dwords], written as packed channel
// pairs and copied out as the one contiguous run it is in memory.  (NCHW output: no tile at all.)
struct NormTile {
  int C, HW;
  int gshift;        // log2 G
  int tiles;         // per image
  int pd;            // dwords per pixel row of the LDS tile (C * sizeof(T) / 4 plus padding)
  int aux;           // float index of the arrays behind the tile
  unsigned mg_cd;    // reciprocal of the dwords per pixel (C * sizeof(T) / 4) for dividends below tp * that (shift 32)
};

template <typename T> struct PairWord;
template <> struct PairWord<bf16_t> {
  static constexpr int kDwords = 1;
  static __device__ __forceinline__ void put(float* tile, int idx, float a, float b) {
    reinterpret_cast<uint32_t*>(tile)[idx] = pack_bf16x2(a, b);
  }
};
template <> struct PairWord<float> {
  static constexpr int kDwords = 2;
  static __device__ __forceinline__ void put(float* tile, int idx, float a, float b) { tile[idx] = a; tile[idx + 1] = b; }
};

template <typename T>
__device__ __forceinline__ void store_quad(T* p, const float (&f)[4]);
template <> __device__ __forceinline__ void store_quad<float>(float* p, const float (&f)[4]) {
  float4 v;
  v.x = f[0]; v.y = f[1]; v.z = f[2]; v.w = f[3];
  *reinterpret_cast<float4*>(p) = v;
}
template <> __device__ __forceinline__ void store_quad<bf16_t>(bf16_t* p, const float (&f)[4]) {
  uint2 v;
  v.x = pack_bf16x2(f[0], f[1]); v.y = pack_bf16x2(f[2], f[3]);
  *reinterpret_cast<uint2*>(p) = v;
}
// VEC: four elements as one aligned vector; else the first n one by one.
template <typename T, bool VEC>
__device__ __forceinline__ void load_row4(Quad<T>& q, const T* p, int n) {
  if constexpr (VEC) q.load(p);
  else q.load_n(p, n);
}
template <typename T, bool VEC>
__device__ __forceinline__ void store_row4(T* p, const float (&f)[4], int n) {
  if constexpr (VEC) {
    store_quad<T>(p, f);
  } else {
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (j < n) p[j] = from_f32<T>(f[j]);
  }
}

// Grid (tiles, B).  NHWC: out is (B, HW, C); else (B, C, HW).
template <typename T, int NP, bool NHWC, bool VEC>
__global__ void __launch_bounds__(kBlockThreads)
channel_norm_reg_kernel(const T* __restrict__ x, T* __restrict__ out, const void* __restrict__ weight,
                        const void* __restrict__ bias, int pdtype, float eps, const NormTile t) {
  WT_SHARED_FLOATS(ldsf);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int G = 1 << t.gshift, tp = 4 * G, cs = kBlockThreads >> t.gshift;
  const int g = tid & (G - 1), e = tid >> t.gshift;
  const int C = t.C, C2 = C >> 1;
  int tile, b;
  tile_of_workgroup(tile, b);
  const int p0 = tile * tp;
  const int np = t.HW - p0 < tp ? t.HW - p0 : tp;
  const int nv = np - 4 * g < 0 ? 0 : (np - 4 * g > 4 ? 4 : np - 4 * g);      // this thread's pixels inside the tile
  const bool live = nv > 0;
  float* psum = ldsf + t.aux;                    // [4 waves][tp]
  float* pvar = psum + 4 * tp;                   // [4 waves][tp]
  float* wgt = pvar + 4 * tp;                    // weight[C], bias[C]
  for (int c = tid; c < C; c += kBlockThreads) {
    wgt[c] = load_param(weight, pdtype, c);
    wgt[C + c] = load_param(bias, pdtype, c);
  }
  const T* src = x + static_cast<size_t>(b) * C * t.HW + p0 + 4 * g;
  Quad<T> q[NP][2];
#pragma unroll
  for (int k = 0; k < NP; ++k) {
    const int cp = e + k * cs;
    if (live && cp < C2) {
      load_row4<T, VEC>(q[k][0], src + static_cast<size_t>(2 * cp) * t.HW, nv);
      load_row4<T, VEC>(q[k][1], src + static_cast<size_t>(2 * cp + 1) * t.HW, nv);
    }
  }
  float v[NP][2][4];
  float s[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int k = 0; k < NP; ++k) {
    const int cp = e + k * cs;
    const bool on = live && cp < C2;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      if (on) q[k][h].get(v[k][h]);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (!on) v[k][h][j] = 0.f;
        s[j] += v[k][h][j];
      }
    }
  }
  // lanes of a wave that share g: lane bits gshift..5
  const int lane4 = lane << 2;
  auto meet = [&](float (&a)[4], float* part) {
    for (int m = 32; m >= G; m >>= 1) {
#pragma unroll
      for (int j = 0; j < 4; ++j) a[j] += wave_xor(a[j], lane4, m);
    }
    if (lane < G) {
#pragma unroll
      for (int j = 0; j < 4; ++j) part[wave * tp + 4 * g + j] = a[j];
    }
  };
  meet(s, psum);
  __syncthreads();                               // (also: wgt is in place)
  const float inv_c = 1.f / static_cast<float>(C);
  float mean[4], sq[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int j = 0; j < 4; ++j)
    mean[j] = (psum[4 * g + j] + psum[tp + 4 * g + j] + psum[2 * tp + 4 * g + j] + psum[3 * tp + 4 * g + j]) * inv_c;
#pragma unroll
  for (int k = 0; k < NP; ++k) {
    const bool on = live && e + k * cs < C2;
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float d = on ? v[k][h][j] - mean[j] : 0.f;
        sq[j] += d * d;
      }
  }
  meet(sq, pvar);
  __syncthreads();
  float rstd[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const float var = (pvar[4 * g + j] + pvar[tp + 4 * g + j] + pvar[2 * tp + 4 * g + j] + pvar[3 * tp + 4 * g + j]) * inv_c;
    rstd[j] = 1.f / sqrtf(var + eps);
  }
  constexpr int PW = PairWord<T>::kDwords;
#pragma unroll
  for (int k = 0; k < NP; ++k) {
    const int cp = e + k * cs;
    if (live && cp < C2) {
      const int c = 2 * cp;
      const float w0 = wgt[c], w1 = wgt[c + 1], b0 = wgt[C + c], b1 = wgt[C + c + 1];
      float y0[4], y1[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        y0[j] = (v[k][0][j] - mean[j]) * rstd[j] * w0 + b0;
        y1[j] = (v[k][1][j] - mean[j]) * rstd[j] * w1 + b1;
      }
      if constexpr (NHWC) {
#pragma unroll
        for (int j = 0; j < 4; ++j) PairWord<T>::put(ldsf, (4 * g + j) * t.pd + cp * PW, y0[j], y1[j]);
      } else {
        T* dst = out + static_cast<size_t>(b) * C * t.HW + p0 + 4 * g;
        store_row4<T, VEC>(dst + static_cast<size_t>(c) * t.HW, y0, nv);
        store_row4<T, VEC>(dst + static_cast<size_t>(c + 1) * t.HW, y1, nv);
      }
    }
  }
  if constexpr (NHWC) {
    __syncthreads();
    // the tile's output is one contiguous run of np * C elements = np * cd dwords
    const int cd = C2 * PW;
    uint32_t* dst = reinterpret_cast<uint32_t*>(out + (static_cast<size_t>(b) * t.HW + p0) * C);
    const uint32_t* tile = reinterpret_cast<const uint32_t*>(ldsf);
    const int total = np * cd;
    constexpr int kBatch = 8;                    // LDS reads a thread has under way before its stores
    for (int i0 = tid; i0 < total; i0 += kBatch * kBlockThreads) {
      uint32_t w[kBatch];
#pragma unroll
      for (int u = 0; u < kBatch; ++u) {
        const int i = i0 + u * kBlockThreads;
        if (i < total) {
          const int pp = div_c(i, t.mg_cd);
          w[u] = tile[pp * t.pd + (i - pp * cd)];
        }
      }
#pragma unroll
      for (int u = 0; u < kBatch; ++u) {
        const int i = i0 + u * kBlockThreads;
        if (i < total) dst[i] = w[u];
      }
    }
  }
}

// Grid (tiles, B).  y is (B, HW, C); shortcut and out are (B, C, HW); gamma may be null (no layer scale).
template <typename T, bool VEC>
__global__ void __launch_bounds__(kBlockThreads)
block_residual_kernel(const T* __restrict__ y, const T* __restrict__ shortcut, const void* __restrict__ gamma,
                      int pdtype, T* __restrict__ out, const BlockTile t) {
  WT_SHARED_FLOATS(ldsf);
  T* lds = reinterpret_cast<T*>(ldsf);
  const int tid = threadIdx.x;
  int tile, b;
  tile_of_workgroup(tile, b);
  const int p0 = tile * t.tp;
  const int pitch = t.tp + 1, C = t.C;
  const int np = t.HW - p0 < t.tp ? t.HW - p0 : t.tp;
  const T* src = y + (static_cast<size_t>(b) * t.HW + p0) * C;
  const int npair = (np * C) >> 1;
  for (int i = tid; i < npair; i += kBlockThreads) {
    const int e = 2 * i;
    const int pp = div_c(e, t.mg_c), c = e - pp * C;
    T a, bb;
    load_pair_raw<T>(src + e, a, bb);
    lds[c * pitch + pp] = a;
    lds[(c + 1) * pitch + pp] = bb;
  }
  __syncthreads();
  if constexpr (VEC) {
    const int gshift = t.tp_shift - 2;
    const int g = tid & ((1 << gshift) - 1), c0 = tid >> gshift, cstep = kBlockThreads >> gshift;
    const int p = 4 * g;
    if (p < np) {
      const size_t base = static_cast<size_t>(b) * C * t.HW + p0 + p;
      for (int cb = c0; cb < C; cb += kQuadBatch * cstep) {
        Quad<T> q[kQuadBatch];
#pragma unroll
        for (int k = 0; k < kQuadBatch; ++k) {
          const int c = cb + k * cstep;
          if (c < C) q[k].load(shortcut + base + static_cast<size_t>(c) * t.HW);
        }
#pragma unroll
        for (int k = 0; k < kQuadBatch; ++k) {
          const int c = cb + k * cstep;
          if (c < C) {
            const float gm = gamma != nullptr ? load_param(gamma, pdtype, c) : 1.f;
            float f[4];
            q[k].get(f);
            T* o = out + base + static_cast<size_t>(c) * t.HW;
            const T* row = lds + c * pitch + p;
            store_pair<T>(o, f[0] + gm * to_f32<T>(row[0]), f[1] + gm * to_f32<T>(row[1]));
            store_pair<T>(o + 2, f[2] + gm * to_f32<T>(row[2]), f[3] + gm * to_f32<T>(row[3]));
          }
        }
      }
    }
  } else {
    const int p = tid & (t.tp - 1), c0 = tid >> t.tp_shift, cstep = kBlockThreads >> t.tp_shift;
    if (p < np) {
      const size_t base = static_cast<size_t>(b) * C * t.HW + p0 + p;
      for (int c = c0; c < C; c += cstep) {
        const float g = gamma != nullptr ? load_param(gamma, pdtype, c) : 1.f;
        const size_t o = base + static_cast<size_t>(c) * t.HW;
        out[o] = from_f32<T>(to_f32<T>(shortcut[o]) + g * to_f32<T>(lds[c * pitch + p]));
      }
    }
  }
}

// The block's second pass on the plan of channel_norm_reg_kernel.  Grid (tiles, B).  The NHWC run of the tile goes into
// LDS as it lies in memory (pixel-major, dword copies); thread (g, e) then takes the channel pairs e, e + cs, ... of
// its four pixels from there as packed words, the shortcut's rows as 4-element vectors straight from HBM (issued before
// the barrier), and writes the rows of the result.
template <typename T> struct PairWordGet;
template <> struct PairWordGet<bf16_t> {
  static __device__ __forceinline__ void get(const float* tile, int idx, float& a, float& b) {
    const uint32_t v = reinterpret_cast<const uint32_t*>(tile)[idx];
    a = __uint_as_float(v << 16); b = __uint_as_float(v & 0xffff0000u);
  }
};
template <> struct PairWordGet<float> {
  static __device__ __forceinline__ void get(const float* tile, int idx, float& a, float& b) { a = tile[idx]; b = tile[idx + 1]; }
};

template <typename T, int NP, bool VEC>
__global__ void __launch_bounds__(kBlockThreads)
block_residual_reg_kernel(const T* __restrict__ y, const T* __restrict__ shortcut, const void* __restrict__ gamma,
                          int pdtype, T* __restrict__ out, const NormTile t) {
  WT_SHARED_FLOATS(ldsf);
  const int tid = threadIdx.x;
  const int G = 1 << t.gshift, tp = 4 * G, cs = kBlockThreads >> t.gshift;
  const int g = tid & (G - 1), e = tid >> t.gshift;
  const int C = t.C, C2 = C >> 1;
  int tile, b;
  tile_of_workgroup(tile, b);
  const int p0 = tile * tp;
  const int np = t.HW - p0 < tp ? t.HW - p0 : tp;
  const int nv = np - 4 * g < 0 ? 0 : (np - 4 * g > 4 ? 4 : np - 4 * g);      // this thread's pixels inside the tile
  const bool live = nv > 0;
  constexpr int PW = PairWord<T>::kDwords;
  const size_t base = static_cast<size_t>(b) * C * t.HW + p0 + 4 * g;
  Quad<T> q[NP][2];
#pragma unroll
  for (int k = 0; k < NP; ++k) {
    const int cp = e + k * cs;
    if (live && cp < C2) {
      load_row4<T, VEC>(q[k][0], shortcut + base + static_cast<size_t>(2 * cp) * t.HW, nv);
      load_row4<T, VEC>(q[k][1], shortcut + base + static_cast<size_t>(2 * cp + 1) * t.HW, nv);
    }
  }
  {
    const int cd = C2 * PW;
    const uint32_t* src = reinterpret_cast<const uint32_t*>(y + (static_cast<size_t>(b) * t.HW + p0) * C);
    uint32_t* tile = reinterpret_cast<uint32_t*>(ldsf);
    const int total = np * cd;
    constexpr int kBatch = 8;                    // loads a thread keeps in flight
    for (int i0 = tid; i0 < total; i0 += kBatch * kBlockThreads) {
      uint32_t w[kBatch];
#pragma unroll
      for (int u = 0; u < kBatch; ++u) {
        const int i = i0 + u * kBlockThreads;
        if (i < total) w[u] = src[i];
      }
#pragma unroll
      for (int u = 0; u < kBatch; ++u) {
        const int i = i0 + u * kBlockThreads;
        if (i < total) {
          const int pp = div_c(i, t.mg_cd);
          tile[pp * t.pd + (i - pp * cd)] = w[u];
        }
      }
    }
  }
  __syncthreads();
#pragma unroll
  for (int k = 0; k < NP; ++k) {
    const int cp = e + k * cs;
    if (live && cp < C2) {
      const int c = 2 * cp;
      const float g0 = gamma != nullptr ? load_param(gamma, pdtype, c) : 1.f;
      const float g1 = gamma != nullptr ? load_param(gamma, pdtype, c + 1) : 1.f;
      float s0[4], s1[4];
      q[k][0].get(s0);
      q[k][1].get(s1);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (VEC || j < nv) {
          float a, bb;
          PairWordGet<T>::get(ldsf, (4 * g + j) * t.pd + cp * PW, a, bb);
          s0[j] += g0 * a;
          s1[j] += g1 * bb;
        }
      }
      store_row4<T, VEC>(out + base + static_cast<size_t>(c) * t.HW, s0, nv);
      store_row4<T, VEC>(out + base + static_cast<size_t>(c + 1) * t.HW, s1, nv);
    }
  }
}

// ------------------------------------------------------------------------------------------ backward passes
// The same two passes under autograd (training keeps the block's structure, wtconvnext/wtconvnext.py:125-140 of the
// reference): tiles as above, two of them per workgroup (the saved input and the incoming gradient), in the tensors'
// own element type.  Parameter gradients are per-workgroup partial sums in the caller's workspace -- record
// (b * tiles + tile) holds NV vectors of C floats -- summed in record order by column_sum_kernel: two fixed stages,
// no atomics.

// LDS [C][tp + 1] -> NCHW rows (pixels past the image are dropped)
template <typename T, bool VEC>
__device__ __forceinline__ void tile_to_nchw(const T* lds, T* __restrict__ img, const BlockTile& t, int p0, int np, int tid) {
  const int pitch = t.tp + 1;
  if constexpr (VEC) {
    const int gshift = t.tp_shift - 2;
    const int g = tid & ((1 << gshift) - 1), c0 = tid >> gshift, cstep = kBlockThreads >> gshift;
    const int p = 4 * g;
    if (p < np)
      for (int c = c0; c < t.C; c += cstep) {
        const T* row = lds + c * pitch + p;
        T* o = img + static_cast<size_t>(c) * t.HW + p0 + p;
        store_pair<T>(o, to_f32<T>(row[0]), to_f32<T>(row[1]));
        store_pair<T>(o + 2, to_f32<T>(row[2]), to_f32<T>(row[3]));
      }
  } else {
    const int p = tid & (t.tp - 1), c0 = tid >> t.tp_shift, cstep = kBlockThreads >> t.tp_shift;
    if (p < np)
      for (int c = c0; c < t.C; c += cstep) img[static_cast<size_t>(c) * t.HW + p0 + p] = lds[c * pitch + p];
  }
}

// NHWC tile (one contiguous run of np * C elements, C even) -> LDS [C][tp + 1]
template <typename T>
__device__ __forceinline__ void tile_from_nhwc(const T* __restrict__ src, T* lds, const BlockTile& t, int np, int tid) {
  const int pitch = t.tp + 1, C = t.C;
  const int npair = (np * C) >> 1;
  for (int i = tid; i < npair; i += kBlockThreads) {
    const int e = 2 * i;
    const int pp = div_c(e, t.mg_c), c = e - pp * C;
    T a, bb;
    load_pair_raw<T>(src + e, a, bb);
    lds[c * pitch + pp] = a;
    lds[(c + 1) * pitch + pp] = bb;
  }
}

// Backward of channel_norm_kernel.  Grid (tiles, B).  x (B, C, HW) is the forward input, dy the gradient of the
// forward output ((B, HW, C) if dy_nhwc else (B, C, HW)), dx (B, C, HW).  Per pixel, with xh = (x - mean) * rstd and
// g = dy * weight:  dx = rstd * (g - mean_c(g) - xh * mean_c(g * xh)).  Per channel: dweight = sum dy * xh,
// dbias = sum dy, left as this workgroup's record {dweight[C], dbias[C]} in `partial`.
template <typename T, bool VEC>
__global__ void __launch_bounds__(kBlockThreads)
channel_norm_bwd_kernel(const T* __restrict__ x, const T* __restrict__ dy, const void* __restrict__ weight, int pdtype,
                        float eps, int dy_nhwc, T* __restrict__ dx, float* __restrict__ partial, const BlockTile t) {
  WT_SHARED_FLOATS(ldsf);
  const int tid = threadIdx.x;
  int tile, b;
  tile_of_workgroup(tile, b);
  const int p0 = tile * t.tp;
  const int pitch = t.tp + 1, C = t.C;
  const int np = t.HW - p0 < t.tp ? t.HW - p0 : t.tp;
  T* xt = reinterpret_cast<T*>(ldsf);            // tile of x, later of dx
  T* gt = xt + C * pitch;                        // tile of dy
  float* psum = ldsf + t.aux;                    // [parts][tp] partial sums (two sets)
  float* pvar = psum + kBlockThreads;
  float* stat = pvar + kBlockThreads;            // mean[tp], rstd[tp], then the two means of the gradient terms
  float* wgt = stat + 4 * t.tp;                  // weight[C]
  const T* ximg = x + static_cast<size_t>(b) * C * t.HW;
  tile_from_nchw<T, T, VEC>(ximg, xt, t, p0, tid);
  if (dy_nhwc) tile_from_nhwc<T>(dy + (static_cast<size_t>(b) * t.HW + p0) * C, gt, t, np, tid);
  else tile_from_nchw<T, T, VEC>(dy + static_cast<size_t>(b) * C * t.HW, gt, t, p0, tid);
  for (int c = tid; c < C; c += kBlockThreads) wgt[c] = load_param(weight, pdtype, c);
  __syncthreads();
  const int p = tid & (t.tp - 1), part_i = tid >> t.tp_shift, parts = kBlockThreads >> t.tp_shift;
  const bool live = p < np;
  const float invC = 1.f / static_cast<float>(C);
  float s = 0.f;
  if (live)
    for (int c = part_i; c < C; c += parts) s += to_f32<T>(xt[c * pitch + p]);
  psum[part_i * t.tp + p] = s;
  __syncthreads();
  float mean = 0.f;
  for (int k = 0; k < parts; ++k) mean += psum[k * t.tp + p];
  mean *= invC;
  float v = 0.f;
  if (live)
    for (int c = part_i; c < C; c += parts) {
      const float d = to_f32<T>(xt[c * pitch + p]) - mean;
      v += d * d;
    }
  pvar[part_i * t.tp + p] = v;
  __syncthreads();
  float var = 0.f;
  for (int k = 0; k < parts; ++k) var += pvar[k * t.tp + p];
  const float rstd = 1.f / sqrtf(var * invC + eps);
  __syncthreads();                               // psum / pvar are reused below
  float s1 = 0.f, s2 = 0.f;
  if (live)
    for (int c = part_i; c < C; c += parts) {
      const float g = to_f32<T>(gt[c * pitch + p]) * wgt[c];
      const float xh = (to_f32<T>(xt[c * pitch + p]) - mean) * rstd;
      s1 += g;
      s2 = fmaf(g, xh, s2);
    }
  psum[part_i * t.tp + p] = s1;
  pvar[part_i * t.tp + p] = s2;
  if (part_i == 0) { stat[p] = mean; stat[t.tp + p] = rstd; }
  __syncthreads();
  float m1 = 0.f, m2 = 0.f;
  for (int k = 0; k < parts; ++k) { m1 += psum[k * t.tp + p]; m2 += pvar[k * t.tp + p]; }
  m1 *= invC; m2 *= invC;
  // per-channel sums over the tile's pixels (before x's tile is overwritten with dx)
  float* rec = partial + (static_cast<size_t>(b) * gridDim.x + tile) * 2 * C;
  for (int c = tid; c < C; c += kBlockThreads) {
    float dw = 0.f, db = 0.f;
    for (int pp = 0; pp < np; ++pp) {
      const float d = to_f32<T>(gt[c * pitch + pp]);
      const float xh = (to_f32<T>(xt[c * pitch + pp]) - stat[pp]) * stat[t.tp + pp];
      dw = fmaf(d, xh, dw);
      db += d;
    }
    rec[c] = dw;
    rec[C + c] = db;
  }
  __syncthreads();
  if (live)
    for (int c = part_i; c < C; c += parts) {
      const float g = to_f32<T>(gt[c * pitch + p]) * wgt[c];
      const float xh = (to_f32<T>(xt[c * pitch + p]) - mean) * rstd;
      xt[c * pitch + p] = from_f32<T>(rstd * (g - m1 - xh * m2));
    }
  __syncthreads();
  tile_to_nchw<T, VEC>(xt, dx + static_cast<size_t>(b) * C * t.HW, t, p0, np, tid);
}

// Backward of block_residual_kernel with a layer scale.  Grid (tiles, B).  dout (B, C, HW) is the gradient of the
// block's output (the shortcut's gradient is dout itself), y (B, HW, C) the forward's NHWC input; dy (B, HW, C) =
// gamma[c] * dout; this workgroup's record in `partial` = dgamma[C] = sum over its pixels of dout * y.
template <typename T, bool VEC>
__global__ void __launch_bounds__(kBlockThreads)
block_residual_bwd_kernel(const T* __restrict__ dout, const T* __restrict__ y, const void* __restrict__ gamma, int pdtype,
                          T* __restrict__ dy, float* __restrict__ partial, const BlockTile t) {
  WT_SHARED_FLOATS(ldsf);
  const int tid = threadIdx.x;
  int tile, b;
  tile_of_workgroup(tile, b);
  const int p0 = tile * t.tp;
  const int pitch = t.tp + 1, C = t.C;
  const int np = t.HW - p0 < t.tp ? t.HW - p0 : t.tp;
  T* dt = reinterpret_cast<T*>(ldsf);            // tile of dout
  T* yt = dt + C * pitch;                        // tile of y
  float* wgt = ldsf + t.aux;                     // gamma[C]
  tile_from_nchw<T, T, VEC>(dout + static_cast<size_t>(b) * C * t.HW, dt, t, p0, tid);
  const size_t run = (static_cast<size_t>(b) * t.HW + p0) * C;
  tile_from_nhwc<T>(y + run, yt, t, np, tid);
  for (int c = tid; c < C; c += kBlockThreads) wgt[c] = load_param(gamma, pdtype, c);
  __syncthreads();
  float* rec = partial + (static_cast<size_t>(b) * gridDim.x + tile) * C;
  for (int c = tid; c < C; c += kBlockThreads) {
    float dg = 0.f;
    for (int pp = 0; pp < np; ++pp) dg = fmaf(to_f32<T>(dt[c * pitch + pp]), to_f32<T>(yt[c * pitch + pp]), dg);
    rec[c] = dg;
  }
  T* dst = dy + run;
  const int npair = (np * C) >> 1;
  for (int i = tid; i < npair; i += kBlockThreads) {
    const int e = 2 * i;
    const int pp = div_c(e, t.mg_c), c = e - pp * C;
    store_pair<T>(dst + e, wgt[c] * to_f32<T>(dt[c * pitch + pp]), wgt[c + 1] * to_f32<T>(dt[(c + 1) * pitch + pp]));
  }
}

// ---- backward passes on the plan of channel_norm_reg_kernel (rows of whole 4-element vectors) ---------------------------
// Sum of `v` over the G = 2^gshift lanes that differ in their low lane bits (the pixel groups of one channel pair);
// every lane of the group gets the total.  DPP within rows of 16 lanes, one cross-lane exchange for G = 32.
__device__ __forceinline__ float group_sum(float v, int gshift, int lane4) {
#ifdef WT_EMULATE
  (void)lane4;
  for (int m = 1; m < (1 << gshift); m <<= 1) v += __shfl_xor(v, m, kWave);
  return v;
#else
  auto dpp = [](float x, auto ctrl) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), decltype(ctrl)::value, 0xf, 0xf, false));
  };
  using std::integral_constant;
  if (gshift >= 1) v += dpp(v, integral_constant<int, 0xB1>{});     // quad_perm [1,0,3,2]
  if (gshift >= 2) v += dpp(v, integral_constant<int, 0x4E>{});     // quad_perm [2,3,0,1]
  if (gshift >= 3) v += dpp(v, integral_constant<int, 0x141>{});    // row_half_mirror
  if (gshift >= 4) v += dpp(v, integral_constant<int, 0x140>{});    // row_mirror
  if (gshift >= 5) v += wave_xor(v, lane4, 16);
  return v;
#endif
}

// A contiguous run of `total` dwords -> the pixel-major LDS tile (rows of cd dwords at a pitch of pd), eight loads in
// flight per thread; and back.
__device__ __forceinline__ void tile_from_run(const uint32_t* __restrict__ src, uint32_t* tile, int total, int cd,
                                              const NormTile& t, int tid) {
  constexpr int kBatch = 8;
  for (int i0 = tid; i0 < total; i0 += kBatch * kBlockThreads) {
    uint32_t w[kBatch];
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      const int i = i0 + u * kBlockThreads;
      if (i < total) w[u] = src[i];
    }
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      const int i = i0 + u * kBlockThreads;
      if (i < total) {
        const int pp = div_c(i, t.mg_cd);
        tile[pp * t.pd + (i - pp * cd)] = w[u];
      }
    }
  }
}
__device__ __forceinline__ void tile_to_run(const uint32_t* tile, uint32_t* __restrict__ dst, int total, int cd,
                                            const NormTile& t, int tid) {
  constexpr int kBatch = 8;
  for (int i0 = tid; i0 < total; i0 += kBatch * kBlockThreads) {
    uint32_t w[kBatch];
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      const int i = i0 + u * kBlockThreads;
      if (i < total) {
        const int pp = div_c(i, t.mg_cd);
        w[u] = tile[pp * t.pd + (i - pp * cd)];
      }
    }
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      const int i = i0 + u * kBlockThreads;
      if (i < total) dst[i] = w[u];
    }
  }
}

// Backward of the channel norm, values in registers.  Grid (tiles, B); arguments as channel_norm_bwd_kernel.  The
// gradient arrives as rows (NCHW: straight into registers) or as the tile's contiguous NHWC run (through the LDS tile,
// read back as packed channel pairs).  Four sums per pixel (x, squared deviations, g, g * xh) meet as in the forward
// kernel; the per-channel sums over the tile's pixels meet across the pixel groups with group_sum.
template <typename T, int NP, bool DY_NHWC, bool VEC>
__global__ void __launch_bounds__(kBlockThreads)
channel_norm_bwd_reg_kernel(const T* __restrict__ x, const T* __restrict__ dy, const void* __restrict__ weight,
                            int pdtype, float eps, T* __restrict__ dx, float* __restrict__ partial, const NormTile t,
                            unsigned* __restrict__ zero_words, int nzero) {
  WT_SHARED_FLOATS(ldsf);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  if (blockIdx.x == 0 && blockIdx.y == 0)        // the tickets of the column sum that follows on the stream
    for (int i = tid; i < nzero; i += kBlockThreads) zero_words[i] = 0u;
  const int G = 1 << t.gshift, tp = 4 * G, cs = kBlockThreads >> t.gshift;
  const int g = tid & (G - 1), e = tid >> t.gshift;
  const int C = t.C, C2 = C >> 1;
  int tile, b;
  tile_of_workgroup(tile, b);
  const int p0 = tile * tp;
  const int np = t.HW - p0 < tp ? t.HW - p0 : tp;
  const int nv = np - 4 * g < 0 ? 0 : (np - 4 * g > 4 ? 4 : np - 4 * g);      // this thread's pixels inside the tile
  const bool live = nv > 0;
  constexpr int PW = PairWord<T>::kDwords;
  float* part = ldsf + t.aux;                    // four arrays [4 waves][tp]
  float* wgt = part + 16 * tp;                   // weight[C]
  for (int c = tid; c < C; c += kBlockThreads) wgt[c] = load_param(weight, pdtype, c);
  const size_t base = static_cast<size_t>(b) * C * t.HW + p0 + 4 * g;
  Quad<T> q[NP][2];
  Quad<T> qd[DY_NHWC ? 1 : NP][2];
#pragma unroll
  for (int k = 0; k < NP; ++k) {
    const int cp = e + k * cs;
    if (live && cp < C2) {
      load_row4<T, VEC>(q[k][0], x + base + static_cast<size_t>(2 * cp) * t.HW, nv);
      load_row4<T, VEC>(q[k][1], x + base + static_cast<size_t>(2 * cp + 1) * t.HW, nv);
      if constexpr (!DY_NHWC) {
        load_row4<T, VEC>(qd[k][0], dy + base + static_cast<size_t>(2 * cp) * t.HW, nv);
        load_row4<T, VEC>(qd[k][1], dy + base + static_cast<size_t>(2 * cp + 1) * t.HW, nv);
      }
    }
  }
  const int cd = C2 * PW;
  if constexpr (DY_NHWC)
    tile_from_run(reinterpret_cast<const uint32_t*>(dy + (static_cast<size_t>(b) * t.HW + p0) * C),
                  reinterpret_cast<uint32_t*>(ldsf), np * cd, cd, t, tid);
  float v[NP][2][4];
  float s[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int k = 0; k < NP; ++k) {
    const bool on = live && e + k * cs < C2;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      if (on) q[k][h].get(v[k][h]);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (!on) v[k][h][j] = 0.f;
        s[j] += v[k][h][j];
      }
    }
  }
  const int lane4 = lane << 2;
  auto meet = [&](float (&a)[4], float* arr) {
    for (int m = 32; m >= G; m >>= 1) {
#pragma unroll
      for (int j = 0; j < 4; ++j) a[j] += wave_xor(a[j], lane4, m);
    }
    if (lane < G) {
#pragma unroll
      for (int j = 0; j < 4; ++j) arr[wave * tp + 4 * g + j] = a[j];
    }
  };
  auto total = [&](const float* arr, int j) {
    return arr[4 * g + j] + arr[tp + 4 * g + j] + arr[2 * tp + 4 * g + j] + arr[3 * tp + 4 * g + j];
  };
  meet(s, part);
  __syncthreads();                               // (also: the weights and the gradient tile are in place)
  const float inv_c = 1.f / static_cast<float>(C);
  float mean[4], sq[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int j = 0; j < 4; ++j) mean[j] = total(part, j) * inv_c;
#pragma unroll
  for (int k = 0; k < NP; ++k) {
    const bool on = live && e + k * cs < C2;
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float d = on ? v[k][h][j] - mean[j] : 0.f;
        v[k][h][j] = d;                          // from here on: deviations
        sq[j] += d * d;
      }
  }
  meet(sq, part + 4 * tp);
  __syncthreads();
  float rstd[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) rstd[j] = 1.f / sqrtf(total(part + 4 * tp, j) * inv_c + eps);
  // the gradient of this thread's values: (d0, d1) of pixel j, channel pair k
  auto grad_pair = [&](int k, int j, float& d0, float& d1) {
    if constexpr (DY_NHWC) {
      PairWordGet<T>::get(ldsf, (4 * g + j) * t.pd + (e + k * cs) * PW, d0, d1);
    } else {
      float f0[4], f1[4];
      qd[k][0].get(f0);
      qd[k][1].get(f1);
      d0 = f0[j]; d1 = f1[j];
    }
  };
  float a1[4] = {0.f, 0.f, 0.f, 0.f}, a2[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int k = 0; k < NP; ++k) {
    const int cp = e + k * cs;
    if (live && cp < C2) {
      const float w0 = wgt[2 * cp], w1 = wgt[2 * cp + 1];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (VEC || j < nv) {                              // (tile rows past the image hold nothing)
          float d0, d1;
          grad_pair(k, j, d0, d1);
          const float g0 = d0 * w0, g1 = d1 * w1;
          a1[j] += g0 + g1;
          a2[j] += (g0 * v[k][0][j] + g1 * v[k][1][j]) * rstd[j];
        }
      }
    }
  }
  meet(a1, part + 8 * tp);
  meet(a2, part + 12 * tp);
  __syncthreads();
  float m1[4], m2[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    m1[j] = total(part + 8 * tp, j) * inv_c;
    m2[j] = total(part + 12 * tp, j) * inv_c;
  }
  float* rec = partial + (static_cast<size_t>(b) * gridDim.x + tile) * 2 * C;
#pragma unroll
  for (int k = 0; k < NP; ++k) {
    const int cp = e + k * cs;
    const bool on = live && cp < C2;
    float dw0 = 0.f, dw1 = 0.f, db0 = 0.f, db1 = 0.f;
    if (on) {
      const float w0 = wgt[2 * cp], w1 = wgt[2 * cp + 1];
      float o0[4] = {0.f, 0.f, 0.f, 0.f}, o1[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (VEC || j < nv) {
          float d0, d1;
          grad_pair(k, j, d0, d1);
          const float xh0 = v[k][0][j] * rstd[j], xh1 = v[k][1][j] * rstd[j];
          o0[j] = rstd[j] * (d0 * w0 - m1[j] - xh0 * m2[j]);
          o1[j] = rstd[j] * (d1 * w1 - m1[j] - xh1 * m2[j]);
          dw0 += d0 * xh0; dw1 += d1 * xh1;
          db0 += d0; db1 += d1;
        }
      }
      store_row4<T, VEC>(dx + base + static_cast<size_t>(2 * cp) * t.HW, o0, nv);
      store_row4<T, VEC>(dx + base + static_cast<size_t>(2 * cp + 1) * t.HW, o1, nv);
    }
    dw0 = group_sum(dw0, t.gshift, lane4); dw1 = group_sum(dw1, t.gshift, lane4);
    db0 = group_sum(db0, t.gshift, lane4); db1 = group_sum(db1, t.gshift, lane4);
    if (g == 0 && cp < C2) {
      rec[2 * cp] = dw0; rec[2 * cp + 1] = dw1;
      rec[C + 2 * cp] = db0; rec[C + 2 * cp + 1] = db1;
    }
  }
}

// Backward of the block residual on the same plan.  Grid (tiles, B); arguments as block_residual_bwd_kernel.  The NHWC
// run of y goes through the LDS tile; each thread replaces the words it reads there by gamma * dout, and the tile leaves
// as the contiguous run of dy.
template <typename T, int NP, bool VEC>
__global__ void __launch_bounds__(kBlockThreads)
block_residual_bwd_reg_kernel(const T* __restrict__ dout, const T* __restrict__ y, const void* __restrict__ gamma,
                              int pdtype, T* __restrict__ dy, float* __restrict__ partial, const NormTile t,
                              unsigned* __restrict__ zero_words, int nzero) {
  WT_SHARED_FLOATS(ldsf);
  const int tid = threadIdx.x, lane = tid & 63;
  if (blockIdx.x == 0 && blockIdx.y == 0)        // the tickets of the column sum that follows on the stream
    for (int i = tid; i < nzero; i += kBlockThreads) zero_words[i] = 0u;
  const int G = 1 << t.gshift, tp = 4 * G, cs = kBlockThreads >> t.gshift;
  const int g = tid & (G - 1), e = tid >> t.gshift;
  const int C = t.C, C2 = C >> 1;
  int tile, b;
  tile_of_workgroup(tile, b);
  const int p0 = tile * tp;
  const int np = t.HW - p0 < tp ? t.HW - p0 : tp;
  const int nv = np - 4 * g < 0 ? 0 : (np - 4 * g > 4 ? 4 : np - 4 * g);      // this thread's pixels inside the tile
  const bool live = nv > 0;
  constexpr int PW = PairWord<T>::kDwords;
  const size_t base = static_cast<size_t>(b) * C * t.HW + p0 + 4 * g;
  Quad<T> q[NP][2];
#pragma unroll
  for (int k = 0; k < NP; ++k) {
    const int cp = e + k * cs;
    if (live && cp < C2) {
      load_row4<T, VEC>(q[k][0], dout + base + static_cast<size_t>(2 * cp) * t.HW, nv);
      load_row4<T, VEC>(q[k][1], dout + base + static_cast<size_t>(2 * cp + 1) * t.HW, nv);
    }
  }
  const int cd = C2 * PW;
  const size_t run = (static_cast<size_t>(b) * t.HW + p0) * C;
  tile_from_run(reinterpret_cast<const uint32_t*>(y + run), reinterpret_cast<uint32_t*>(ldsf), np * cd, cd, t, tid);
  __syncthreads();
  const int lane4 = lane << 2;
  float* rec = partial + (static_cast<size_t>(b) * gridDim.x + tile) * C;
#pragma unroll
  for (int k = 0; k < NP; ++k) {
    const int cp = e + k * cs;
    float dg0 = 0.f, dg1 = 0.f;
    if (live && cp < C2) {
      const float g0 = load_param(gamma, pdtype, 2 * cp), g1 = load_param(gamma, pdtype, 2 * cp + 1);
      float d0[4], d1[4];
      q[k][0].get(d0);
      q[k][1].get(d1);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (VEC || j < nv) {
          const int idx = (4 * g + j) * t.pd + cp * PW;
          float ya, yb;
          PairWordGet<T>::get(ldsf, idx, ya, yb);
          dg0 += d0[j] * ya;
          dg1 += d1[j] * yb;
          PairWord<T>::put(ldsf, idx, g0 * d0[j], g1 * d1[j]);
        }
      }
    }
    dg0 = group_sum(dg0, t.gshift, lane4);
    dg1 = group_sum(dg1, t.gshift, lane4);
    if (g == 0 && cp < C2) { rec[2 * cp] = dg0; rec[2 * cp + 1] = dg1; }
  }
  __syncthreads();
  tile_to_run(reinterpret_cast<const uint32_t*>(ldsf), reinterpret_cast<uint32_t*>(dy + run), np * cd, cd, t, tid);
}

// out[v] = sum over the `nrec` records of partial[r][v], v < ncol, added in record order (grid = ceil(ncol / 64)
// workgroups of 256 threads: four row groups per column, joined through LDS in a fixed order).
__global__ void __launch_bounds__(kBlockThreads) column_sum_kernel(const float* __restrict__ partial, int nrec, int ncol,
                                                                   float* __restrict__ out0, float* __restrict__ out1,
                                                                   int split) {
  __shared__ float red[kBlockThreads];
  const int col = blockIdx.x * 64 + (threadIdx.x & 63), grp = threadIdx.x >> 6;
  float s = 0.f;
  if (col < ncol) {
    const int per = (nrec + 3) / 4;
    const int r0 = grp * per, r1 = r0 + per < nrec ? r0 + per : nrec;
#pragma unroll 4
    for (int r = r0; r < r1; ++r) s += partial[static_cast<size_t>(r) * ncol + col];
  }
  red[threadIdx.x] = s;
  __syncthreads();
  if (grp == 0 && col < ncol) {
    const float v = (red[threadIdx.x] + red[threadIdx.x + 64]) + (red[threadIdx.x + 128] + red[threadIdx.x + 192]);
    if (col < split) out0[col] = v;
    else out1[col - split] = v;
  }
}

// The same sum for many records, in two fixed stages inside one launch.  Grid (ceil(ncol / 64), ns): workgroup
// (cb, s) sums the records of slice s (contiguous, ceil(nrec / ns) of them) for its 64 columns and leaves the result in
// slices[s][col]; the workgroup of a column block that finishes last adds the ns slice sums in slice order.  `tickets`:
// one zeroed word per column block (left zero again).
__global__ void __launch_bounds__(kBlockThreads)
column_sum_sliced_kernel(const float* __restrict__ partial, int nrec, int ncol, float* __restrict__ slices,
                         unsigned* __restrict__ tickets, float* __restrict__ out0, float* __restrict__ out1, int split) {
  __shared__ float red[kBlockThreads];
  __shared__ unsigned flag;
  const int col = blockIdx.x * 64 + (threadIdx.x & 63), grp = threadIdx.x >> 6;
  const int ns = gridDim.y, sl = blockIdx.y;
  const int per = (nrec + ns - 1) / ns;
  const int rb = sl * per, re = rb + per < nrec ? rb + per : nrec;
  float s = 0.f;
  if (col < ncol && rb < re) {
    const int per_g = (re - rb + 3) / 4;
    const int r0 = rb + grp * per_g, r1 = r0 + per_g < re ? r0 + per_g : re;
#pragma unroll 8
    for (int r = r0; r < r1; ++r) s += partial[static_cast<size_t>(r) * ncol + col];
  }
  red[threadIdx.x] = s;
  __syncthreads();
  if (grp == 0 && col < ncol) {
    const float v = (red[threadIdx.x] + red[threadIdx.x + 64]) + (red[threadIdx.x + 128] + red[threadIdx.x + 192]);
    store_shared_f32(slices + static_cast<size_t>(sl) * ncol + col, v);
  }
  if (workgroup_is_last(tickets + blockIdx.x, static_cast<unsigned>(ns), &flag)) {
    if (grp == 0 && col < ncol) {
      float v = 0.f;
      for (int q0 = 0; q0 < ns; q0 += 8) {       // eight loads under way, added in slice order
        float w[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) w[u] = q0 + u < ns ? load_shared_f32(slices + static_cast<size_t>(q0 + u) * ncol + col) : 0.f;
#pragma unroll
        for (int u = 0; u < 8; ++u) v += w[u];
      }
      if (col < split) out0[col] = v;
      else out1[col - split] = v;
    }
    if (threadIdx.x == 0) tickets[blockIdx.x] = 0u;
  }
}

}  // namespace wt
