// Level-by-level WTConv2d kernels for planes whose pyramid does not fit the 160 KB of LDS of
// a compute unit (e.g. 128x128 and larger): every level of the pyramid goes through an fp32
// workspace in HBM, and each kernel works on 16x16 tiles staged in LDS with a halo of R.
// Same maths as kernels2d.h (reference wtconv/wtconv2d.py:38-87, wtconv/util/wavelet.py:62-75);
// about three times the HBM traffic of the plane-resident kernels, any plane size.
//
// Workspace layout (floats), n = B*C planes:
//   A_l, l = 1..L : [n][4][h_l][w_l]     sub-bands LL, LH, HL, HH of level l
//   Z_l, l = 2..L : [n][h_{l-1}][w_{l-1}] reconstruction of level l (added to the LL band of l-1)
#pragma once

#include "common.h"

namespace wt {

constexpr int kStreamTile = 16;     // coefficients per tile edge; 256 threads, one each

struct Stream2D {
  int C, H, W, L, nplanes;
  int h[kMaxLevels + 1], w[kMaxLevels + 1];
  size_t aoff[kMaxLevels + 1];      // A_l (l >= 1), floats from the start of the pyramid area
  size_t zoff[kMaxLevels + 2];      // Z_l (l >= 2)
  size_t floats;                    // whole pyramid area
};

// One analysis level: src = x / grad_out (element type TS) or the LL band of the level above
// (fp32, plane stride 4*hs*ws); reading one past an odd source size returns the zero padding
// the reference applies (wtconv2d.py:49-51).  grid = (tiles, planes <= 65535), block = 256.
template <typename TS>
__global__ void stream_analysis_kernel(const TS* __restrict__ src, size_t src_plane_stride, int hs, int ws,
                                       float* __restrict__ dst, int hd, int wd, int nplanes) {
  const int n = hd * wd;
  for (int plane = blockIdx.y; plane < nplanes; plane += gridDim.y) {
    const TS* s = src + static_cast<size_t>(plane) * src_plane_stride;
    float* d = dst + static_cast<size_t>(plane) * 4 * n;
    for (int q = blockIdx.x * blockDim.x + threadIdx.x; q < n; q += gridDim.x * blockDim.x) {
      const int i = q / wd, j = q - i * wd;
      const bool r1 = 2 * i + 1 < hs, c1 = 2 * j + 1 < ws;
      const TS* p = s + static_cast<size_t>(2 * i) * ws + 2 * j;
      const float a = to_f32<TS>(p[0]);
      const float b = c1 ? to_f32<TS>(p[1]) : 0.f;
      const float c = r1 ? to_f32<TS>(p[ws]) : 0.f;
      const float e = (r1 && c1) ? to_f32<TS>(p[ws + 1]) : 0.f;
      const float sac = a + c, sbd = b + e, dac = a - c, dbd = b - e;
      d[q] = 0.5f * (sac + sbd);
      d[n + q] = 0.5f * (dac + dbd);
      d[2 * n + q] = 0.5f * (sac - sbd);
      d[3 * n + q] = 0.5f * (dac - dbd);
    }
  }
}

// Synthesis of level l: the four sub-band convs of a 16x16 tile of coefficients, + Z_{l+1},
// inverse Haar, cropped.  FINAL (l = 1) adds the scaled base conv and bias of the 32x32
// pixels and stores the layer output; otherwise the result goes to Z_l.
// grid = (tiles_x * tiles_y, planes <= 65535), block = 256.
template <typename T, int K, bool FINAL>
__global__ __launch_bounds__(256) void stream_synth_kernel(const float* __restrict__ A, int hl, int wl,
                                                           const float* __restrict__ Zin,
                                                           float* __restrict__ Zout, int ho, int wo,
                                                           const T* __restrict__ x, T* __restrict__ out,
                                                           const float* __restrict__ fw,
                                                           const float* __restrict__ fb, int C, int NF, int f0,
                                                           int nplanes) {
  constexpr int R = K / 2;
  constexpr int TS = kStreamTile;
  constexpr int AW = TS + 2 * R;            // haloed tile edge
  constexpr int XW = 2 * TS + 2 * R;
  __shared__ float At[4][AW][AW];
  __shared__ float Xt[FINAL ? XW : 1][FINAL ? XW : 1];
  const int tiles_x = (wl + TS - 1) / TS;
  const int ty = blockIdx.x / tiles_x, tx = blockIdx.x - ty * tiles_x;
  const int i0 = ty * TS, j0 = tx * TS;
  const int tid = threadIdx.x;
  const int r = tid / TS, c = tid - r * TS;
  const size_t n = static_cast<size_t>(hl) * wl;
  for (int pv = blockIdx.y; pv < nplanes; pv += gridDim.y) {
    const int plane = WT_UNIFORM(pv);
    const int ch = plane % C;
    const float* Ap = A + static_cast<size_t>(plane) * 4 * n;
    for (int e = tid; e < 4 * AW * AW; e += 256) {
      const int s = e / (AW * AW), rem = e - s * AW * AW;
      const int rr = rem / AW, cc = rem - rr * AW;
      const int gi = i0 + rr - R, gj = j0 + cc - R;
      At[s][rr][cc] = (gi >= 0 && gi < hl && gj >= 0 && gj < wl) ? Ap[s * n + static_cast<size_t>(gi) * wl + gj] : 0.f;
    }
    if constexpr (FINAL) {
      const T* xp = x + static_cast<size_t>(plane) * ho * wo;
      for (int e = tid; e < XW * XW; e += 256) {
        const int rr = e / XW, cc = e - rr * XW;
        const int gi = 2 * i0 + rr - R, gj = 2 * j0 + cc - R;
        Xt[rr][cc] = (gi >= 0 && gi < ho && gj >= 0 && gj < wo) ? to_f32<T>(xp[static_cast<size_t>(gi) * wo + gj]) : 0.f;
      }
    }
    __syncthreads();
    const int i = i0 + r, j = j0 + c;
    if (i < hl && j < wl) {
      wt_uniform_ptr fwc = (wt_uniform_ptr)(fw + static_cast<size_t>(ch) * NF * K * K);
      float y[4];
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        wt_uniform_ptr w = fwc + (f0 + s) * K * K;
        float acc = 0.f;
#pragma unroll
        for (int kh = 0; kh < K; ++kh)
#pragma unroll
          for (int kw = 0; kw < K; ++kw) acc = fmaf(w[kh * K + kw], At[s][r + kh][c + kw], acc);
        y[s] = acc;
      }
      if (Zin != nullptr) y[0] += Zin[static_cast<size_t>(plane) * n + static_cast<size_t>(i) * wl + j];
      const float p = y[0] + y[1], m = y[0] - y[1], q = y[2] + y[3], d = y[2] - y[3];
      float o[2][2] = {{0.5f * (p + q), 0.5f * (p - q)}, {0.5f * (m + d), 0.5f * (m - d)}};
      if constexpr (FINAL) {
        wt_uniform_ptr wb = fwc;
        const float bias = fb[ch];
#pragma unroll
        for (int dr = 0; dr < 2; ++dr)
#pragma unroll
          for (int dc = 0; dc < 2; ++dc) {
            float acc = bias;
#pragma unroll
            for (int kh = 0; kh < K; ++kh)
#pragma unroll
              for (int kw = 0; kw < K; ++kw)
                acc = fmaf(wb[kh * K + kw], Xt[2 * r + dr + kh][2 * c + dc + kw], acc);
            o[dr][dc] += acc;
          }
      }
#pragma unroll
      for (int dr = 0; dr < 2; ++dr)
#pragma unroll
        for (int dc = 0; dc < 2; ++dc) {
          const int oi = 2 * i + dr, oj = 2 * j + dc;
          if (oi < ho && oj < wo) {
            const size_t at = static_cast<size_t>(plane) * ho * wo + static_cast<size_t>(oi) * wo + oj;
            if constexpr (FINAL) out[at] = from_f32<T>(o[dr][dc]);
            else Zout[at] = o[dr][dc];
          }
        }
    }
    __syncthreads();
  }
}

// Correlation sums of one filter set: dWt[kh][kw] = sum_{b,i,j} G[i][j] * A[i+kh-R][j+kw-R]
// over the batch items of a chunk.  grid = (C * nsub, nchunk), block = 256; blockIdx.x =
// c * nsub + s.  A and G: element type TS, plane (b, c) at plane * plane_stride + s * sub_stride,
// h x w each.  Results: partial[(chunk * C + c) * rec + (f0 + s) * K*K + t], and the plain sum of
// G at partial[... + rec - 1] when `with_gsum` (base conv: the bias gradient).
template <typename TS, int K>
__global__ __launch_bounds__(256) void stream_corr_kernel(const TS* __restrict__ A, const TS* __restrict__ G,
                                                          size_t plane_stride, size_t sub_stride, int h, int w,
                                                          float* __restrict__ partial, int rec, int f0, int nsub,
                                                          int with_gsum, int B, int C, int bchunk) {
  constexpr int R = K / 2;
  constexpr int TS_ = kStreamTile;
  constexpr int AW = TS_ + 2 * R;
  constexpr int KK = K * K;
  __shared__ float At[AW][AW];
  __shared__ float Gt[TS_][TS_];
  __shared__ float red[4][KK + 1];
  const int cc = blockIdx.x / nsub, s = blockIdx.x - cc * nsub;
  const int chunk = blockIdx.y;
  const int tid = threadIdx.x;
  const int r = tid / TS_, c = tid - r * TS_;
  const int tiles_x = (w + TS_ - 1) / TS_, tiles_y = (h + TS_ - 1) / TS_;
  float acc[KK];
  float gsum = 0.f;
#pragma unroll
  for (int t = 0; t < KK; ++t) acc[t] = 0.f;
  const int b_end = (chunk + 1) * bchunk < B ? (chunk + 1) * bchunk : B;
  for (int b = chunk * bchunk; b < b_end; ++b) {
    const size_t base = (static_cast<size_t>(b) * C + cc) * plane_stride + static_cast<size_t>(s) * sub_stride;
    const TS* Ap = A + base;
    const TS* Gp = G + base;
    for (int tile = 0; tile < tiles_x * tiles_y; ++tile) {
      const int ty = tile / tiles_x, tx = tile - ty * tiles_x;
      const int i0 = ty * TS_, j0 = tx * TS_;
      for (int e = tid; e < AW * AW; e += 256) {
        const int rr = e / AW, c2 = e - rr * AW;
        const int gi = i0 + rr - R, gj = j0 + c2 - R;
        At[rr][c2] = (gi >= 0 && gi < h && gj >= 0 && gj < w) ? to_f32<TS>(Ap[static_cast<size_t>(gi) * w + gj]) : 0.f;
      }
      {
        const int gi = i0 + r, gj = j0 + c;
        Gt[r][c] = (gi < h && gj < w) ? to_f32<TS>(Gp[static_cast<size_t>(gi) * w + gj]) : 0.f;
      }
      __syncthreads();
      const float gv = Gt[r][c];
      gsum += gv;
#pragma unroll
      for (int kh = 0; kh < K; ++kh)
#pragma unroll
        for (int kw = 0; kw < K; ++kw) acc[kh * K + kw] = fmaf(gv, At[r + kh][c + kw], acc[kh * K + kw]);
      __syncthreads();
    }
  }
  const int wave = tid >> 6, lane = tid & (kWave - 1);
#pragma unroll
  for (int t = 0; t < KK; ++t) {
    const float v = wave_sum(acc[t]);
    if (lane == 0) red[wave][t] = v;
  }
  {
    const float v = wave_sum(gsum);
    if (lane == 0) red[wave][KK] = v;
  }
  __syncthreads();
  float* dst = partial + (static_cast<size_t>(chunk) * C + cc) * rec;
  if (tid < KK) dst[(f0 + s) * KK + tid] = red[0][tid] + red[1][tid] + red[2][tid] + red[3][tid];
  if (with_gsum && tid == KK) dst[rec - 1] = red[0][KK] + red[1][KK] + red[2][KK] + red[3][KK];
}

}  // namespace wt
