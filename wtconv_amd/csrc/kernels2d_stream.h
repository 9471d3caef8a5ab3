// Level-by-level WTConv2d kernels for planes whose pyramid does not fit the 160 KB of LDS of
// a compute unit (e.g. 128x128 and larger): every level of the pyramid goes through an fp32
// workspace in HBM, and each kernel works on tiles of 16 x 64 coefficients staged in LDS with a halo.
// Same maths as kernels2d.h (reference wtconv/wtconv2d.py:38-87, wtconv/util/wavelet.py:62-75);
// about three times the HBM traffic of the plane-resident kernels, any plane size.
//
// Workspace layout (floats), n = B*C planes:
//   A_l, l = 1..L : [n][4][h_l][w_l]     sub-bands LL, LH, HL, HH of level l
//   Z_l, l = 2..L : [n][h_{l-1}][w_{l-1}] reconstruction of level l (added to the LL band of l-1)
#pragma once

#include "common.h"
#include "kernels2d.h"

namespace wt {

constexpr int kStreamTile = 16;     // tile rows (coefficients)
constexpr int kStreamTileW = 64;    // tile columns: 256 threads, four adjacent coefficients each
constexpr int kStreamPad = 4;       // column halo of the LDS tiles (>= K/2, keeps rows 16-byte aligned)

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
template <typename TS, bool LL_ONLY>
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
      if constexpr (!LL_ONLY) {            // the forward pass rebuilds the level-1 detail bands from x itself
        d[n + q] = 0.5f * (dac + dbd);
        d[2 * n + q] = 0.5f * (sac - sbd);
        d[3 * n + q] = 0.5f * (dac - dbd);
      }
    }
  }
}

// Copy of a window of NS stacked planes (plane s at src + s * sub_stride, h x w each) into
// LDS: dst[(s * ROWS + r) * WD + c] = plane_s[gi0 + r][gj0 + c], zero outside the plane.  256
// threads walk the window VW elements at a time (VW = 4: w and gj0 multiples of 4 and src
// aligned to 4 elements); the (s, r, c) position advances without divisions.  `fetch` issues
// all loads of the thread (a compile-time count, so they are in flight together), `commit`
// writes them to LDS; other work can go between the two.
template <typename TS, int NS, int ROWS, int WD, int VW>
struct WindowStage {
  static constexpr int W4 = WD / VW;
  static constexpr int N = NS * ROWS * W4;
  static constexpr int IT = (N + 255) / 256;
  static constexpr int DR = 256 / W4, DC = 256 % W4;
  static_assert(WD % VW == 0 && DR + (DC != 0 ? 1 : 0) <= ROWS, "window too small for the stepping rule");
  float v[IT][VW];

  __device__ __forceinline__ void fetch(const TS* __restrict__ src, size_t sub_stride, int h, int w, int gi0,
                                        int gj0, int tid) {
    int row = tid / W4, col = tid - row * W4;
    int s = row / ROWS, rr = row - s * ROWS;
#pragma unroll
    for (int it = 0; it < IT; ++it) {
      const int gi = gi0 + rr, gj = gj0 + col * VW;
#pragma unroll
      for (int e = 0; e < VW; ++e) v[it][e] = 0.f;
      if (s < NS && gi >= 0 && gi < h && gj >= 0 && gj < w) {
        const TS* q = src + (s * static_cast<int>(sub_stride) + gi * w + gj);   // stacked planes < 2^31 elements
        if constexpr (VW == 4) load4<TS>(q, v[it]);
        else v[it][0] = to_f32<TS>(q[0]);
      }
      col += DC;
      rr += DR;
      if (col >= W4) { col -= W4; ++rr; }
      if (rr >= ROWS) { rr -= ROWS; ++s; }
    }
  }

  __device__ __forceinline__ void commit(float* __restrict__ dst, int tid) const {
    int row = tid / W4, col = tid - row * W4;
#pragma unroll
    for (int it = 0; it < IT; ++it) {
      if (it * 256 + tid < N) {
        float* d = dst + row * WD + col * VW;
        if constexpr (VW == 4) {
          float4 t4;
          t4.x = v[it][0]; t4.y = v[it][1]; t4.z = v[it][2]; t4.w = v[it][3];
          *reinterpret_cast<float4*>(d) = t4;
        } else {
          d[0] = v[it][0];
        }
      }
      col += DC;
      row += DR;
      if (col >= W4) { col -= W4; ++row; }
    }
  }
};

template <typename TS, int NS, int ROWS, int WD, int VW>
__device__ __forceinline__ void stage_window(const TS* __restrict__ src, size_t sub_stride, int h, int w, int gi0,
                                             int gj0, float* __restrict__ dst, int tid) {
  WindowStage<TS, NS, ROWS, WD, VW> st;
  st.fetch(src, sub_stride, h, w, gi0, gj0, tid);
  st.commit(dst, tid);
}

// Twelve floats of an LDS row from a 16-byte aligned address.
__device__ __forceinline__ void lds_read12(const float* __restrict__ p, float (&v)[12]) {
#pragma unroll
  for (int q = 0; q < 3; ++q) {
    const float4 t4 = reinterpret_cast<const float4*>(p)[q];
    v[4 * q] = t4.x; v[4 * q + 1] = t4.y; v[4 * q + 2] = t4.z; v[4 * q + 3] = t4.w;
  }
}

// Tiles of the synthesis kernel.  Levels >= 2: the four sub-bands of the level (haloed, VA
// elements per load) from the pyramid.  Last level: only the input pixels under the haloed
// coefficient tile (VO elements per load); the level-1 sub-bands are rebuilt from them in LDS
// (haar_tile), which saves reading -- and, in the analysis kernel, writing -- three quarters of
// the level-1 pyramid.
template <typename T, int K, bool FINAL, int VA, int VO>
__device__ __forceinline__ void synth_stage_tiles(const float* __restrict__ Ap, size_t n, int hl, int wl,
                                                  const T* __restrict__ xp, int ho, int wo, int i0, int j0,
                                                  float* __restrict__ At, float* __restrict__ Xt, int tid) {
  constexpr int R = K / 2;
  constexpr int TH = kStreamTile, TW = kStreamTileW, HP = kStreamPad;
  if constexpr (FINAL) {
    WindowStage<T, 1, 2 * (TH + 2 * R), 2 * (TW + 2 * HP), VO> sx;
    sx.fetch(xp, 0, ho, wo, 2 * (i0 - R), 2 * (j0 - HP), tid);
    sx.commit(Xt, tid);
  } else {
    WindowStage<float, 4, TH + 2 * R, TW + 2 * HP, VA> sa;
    sa.fetch(Ap, n, hl, wl, i0 - R, j0 - HP, tid);
    sa.commit(At, tid);
  }
}

// Level-1 Haar analysis of a pixel tile in LDS: coefficient (rr, cc) of the AH x AWD tile comes
// from pixels (2rr .. 2rr+1, 2cc .. 2cc+1) of the 2AH x 2AWD pixel tile.  Pixels outside the
// plane were staged as zeros, which is both the zero padding of odd sizes and the zero halo of
// the sub-band convs (a coefficient outside the level has all four pixels outside the plane).
template <int AH, int AWD>
__device__ __forceinline__ void haar_tile(const float* __restrict__ Xt, float* __restrict__ At, int tid) {
  constexpr int XWD = 2 * AWD;
  constexpr int PAIRS = AWD / 2;             // two coefficients (four pixels of each row) per step
  for (int e = tid; e < AH * PAIRS; e += 256) {
    const int rr = e / PAIRS, cp = e - rr * PAIRS;
    const float4 top = *reinterpret_cast<const float4*>(Xt + (2 * rr) * XWD + 4 * cp);
    const float4 bot = *reinterpret_cast<const float4*>(Xt + (2 * rr + 1) * XWD + 4 * cp);
    const float a[2] = {top.x, top.z}, b[2] = {top.y, top.w}, c[2] = {bot.x, bot.z}, d[2] = {bot.y, bot.w};
    float o[4][2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {            // same operation order as stream_analysis_kernel
      const float sac = a[t] + c[t], sbd = b[t] + d[t], dac = a[t] - c[t], dbd = b[t] - d[t];
      o[0][t] = 0.5f * (sac + sbd);
      o[1][t] = 0.5f * (dac + dbd);
      o[2][t] = 0.5f * (sac - sbd);
      o[3][t] = 0.5f * (dac - dbd);
    }
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      float* dst = At + (s * AH + rr) * AWD + 2 * cp;
      dst[0] = o[s][0];
      dst[1] = o[s][1];
    }
  }
}

// Synthesis of level l: the four sub-band convs of a tile of 16 x 64 coefficients, + Z_{l+1},
// inverse Haar, cropped.  FINAL (l = 1) takes its sub-bands from the input pixels (`A` unused),
// adds the scaled base conv and bias of the 32 x 128 pixels and stores the layer output;
// otherwise the sub-bands come from the pyramid and the result goes to Z_l.  A thread owns four
// adjacent coefficients of a row (2 x 8 output pixels): every LDS row it reads as 16-byte
// vectors feeds 4K (sub-bands) or 8K (base conv) products.  The tiles carry a column halo of
// 4 so that their rows start at multiples of 4 elements of the source row.
// `vec`: bit 0 = A / Zin rows can be read as 4-element vectors (wl % 4 == 0, aligned bases),
// bit 1 = x / out / Zout rows likewise (wo % 4 == 0).
// grid = (tiles_x * tiles_y, gy, gz) with gy * gz >= planes, block = 256.
template <typename T, int K, bool FINAL>
__global__ __launch_bounds__(256, 3) void stream_synth_kernel(const float* __restrict__ A, int hl, int wl,
                                                           const float* __restrict__ Zin,
                                                           float* __restrict__ Zout, int ho, int wo,
                                                           const T* __restrict__ x, T* __restrict__ out,
                                                           const float* __restrict__ fw,
                                                           const float* __restrict__ fb, int C, int NF, int f0,
                                                           int nplanes, int vec) {
  constexpr int R = K / 2;
  constexpr int TH = kStreamTile, TW = kStreamTileW, HP = kStreamPad, TJ = 4;
  constexpr int AH = TH + 2 * R, AWD = TW + 2 * HP;
  constexpr int XH = 2 * AH, XWD = 2 * AWD;   // last level: the pixels under the haloed coefficient tile
  __shared__ alignas(16) float At[4 * AH * AWD];
  __shared__ alignas(16) float Xt[FINAL ? XH * XWD : 4];
  const int tiles_x = (wl + TW - 1) / TW;
  const int ty = blockIdx.x / tiles_x, tx = blockIdx.x - ty * tiles_x;
  const int i0 = ty * TH, j0 = tx * TW;
  const int tid = threadIdx.x;
  const int r = tid >> 4, c0 = (tid & 15) * TJ;
  const size_t n = static_cast<size_t>(hl) * wl;
  const bool vec_a = (vec & 1) != 0, vec_o = (vec & 2) != 0;
  {                                          // no loop over planes: nothing to hoist into registers
    const int plane = WT_UNIFORM(static_cast<int>(blockIdx.z * gridDim.y + blockIdx.y));
    if (plane >= nplanes) return;
    const int ch = plane % C;
    const float* Ap = A + static_cast<size_t>(plane) * 4 * n;
    const T* xp = FINAL ? x + static_cast<size_t>(plane) * ho * wo : nullptr;
    if (vec_a) {
      if (vec_o) synth_stage_tiles<T, K, FINAL, 4, 4>(Ap, n, hl, wl, xp, ho, wo, i0, j0, At, Xt, tid);
      else synth_stage_tiles<T, K, FINAL, 4, 1>(Ap, n, hl, wl, xp, ho, wo, i0, j0, At, Xt, tid);
    } else {
      if (vec_o) synth_stage_tiles<T, K, FINAL, 1, 4>(Ap, n, hl, wl, xp, ho, wo, i0, j0, At, Xt, tid);
      else synth_stage_tiles<T, K, FINAL, 1, 1>(Ap, n, hl, wl, xp, ho, wo, i0, j0, At, Xt, tid);
    }
    __syncthreads();
    if constexpr (FINAL) {
      haar_tile<AH, AWD>(Xt, At, tid);
      __syncthreads();
    }
    const int i = i0 + r, j = j0 + c0;
    if (i < hl && j < wl) {
      wt_uniform_ptr fwc = (wt_uniform_ptr)(fw + static_cast<size_t>(ch) * NF * K * K);
      float y[4][TJ];
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        wt_uniform_ptr w = fwc + (f0 + s) * K * K;
#pragma unroll
        for (int t = 0; t < TJ; ++t) y[s][t] = 0.f;
#pragma unroll
        for (int kh = 0; kh < K; ++kh) {
          float v[12];
          lds_read12(At + (s * AH + r + kh) * AWD + c0, v);
#pragma unroll
          for (int kw = 0; kw < K; ++kw)
#pragma unroll
            for (int t = 0; t < TJ; ++t) y[s][t] = fmaf(w[kh * K + kw], v[t + kw - R + HP], y[s][t]);
        }
        WT_CHUNK_FENCE();                    // one sub-band's LDS rows in registers at a time
      }
      if (Zin != nullptr) {
        const float* zp = Zin + static_cast<size_t>(plane) * n + static_cast<size_t>(i) * wl + j;
        if (vec_a) {
          float z[4];
          load4<float>(zp, z);
#pragma unroll
          for (int t = 0; t < TJ; ++t) y[0][t] += z[t];
        } else {
#pragma unroll
          for (int t = 0; t < TJ; ++t)
            if (j + t < wl) y[0][t] += zp[t];
        }
      }
      float o[2][2 * TJ];
#pragma unroll
      for (int t = 0; t < TJ; ++t) {
        const float p = y[0][t] + y[1][t], m = y[0][t] - y[1][t], q = y[2][t] + y[3][t], d = y[2][t] - y[3][t];
        o[0][2 * t] = 0.5f * (p + q);
        o[0][2 * t + 1] = 0.5f * (p - q);
        o[1][2 * t] = 0.5f * (m + d);
        o[1][2 * t + 1] = 0.5f * (m - d);
      }
      if constexpr (FINAL) {
        wt_uniform_ptr wb = fwc;
        const float bias = fb[ch];
#pragma unroll
        for (int u = 0; u < 2 * TJ; ++u) { o[0][u] += bias; o[1][u] += bias; }
#pragma unroll
        for (int xr = 0; xr < K + 1; ++xr) {
          float v[16];
          const float* rowp = Xt + (2 * r + xr + R) * XWD + 2 * c0 + HP;
          {
            float lo[12];
            lds_read12(rowp, lo);
#pragma unroll
            for (int e = 0; e < 12; ++e) v[e] = lo[e];
            const float4 t4 = reinterpret_cast<const float4*>(rowp)[3];
            v[12] = t4.x; v[13] = t4.y; v[14] = t4.z; v[15] = t4.w;
          }
#pragma unroll
          for (int dr = 0; dr < 2; ++dr) {
            const int kh = xr - dr;
            if (kh < 0 || kh >= K) continue;
#pragma unroll
            for (int kw = 0; kw < K; ++kw)
#pragma unroll
              for (int u = 0; u < 2 * TJ; ++u)
                o[dr][u] = fmaf(wb[kh * K + kw], v[u + kw - R + HP], o[dr][u]);
          }
          if (xr & 1) WT_CHUNK_FENCE();      // two input rows in registers at a time
        }
      }
      const int oj = 2 * j;
      const int nvalid = wo - oj < 2 * TJ ? wo - oj : 2 * TJ;
#pragma unroll
      for (int dr = 0; dr < 2; ++dr) {
        const int oi = 2 * i + dr;
        if (oi < ho && nvalid > 0) {
          const size_t at = static_cast<size_t>(plane) * ho * wo + static_cast<size_t>(oi) * wo + oj;
          if constexpr (FINAL) store_row<T, 2 * TJ>(out + at, o[dr], nvalid, vec_o);
          else store_row<float, 2 * TJ>(Zout + at, o[dr], nvalid, vec_o);
        }
      }
    }
  }
}

// Units [u_begin, u_end) of one correlation workgroup; the tiles of unit u + 1 are fetched
// into registers while unit u is multiplied out of LDS.
template <typename TS, int K, int VW>
__device__ __forceinline__ void corr_units(const TS* __restrict__ A, const TS* __restrict__ G, size_t plane_stride,
                                           size_t sub_off, int h, int w, int C, int cc, int tiles_x, int tiles,
                                           int u_begin, int u_end, float* __restrict__ At, float* __restrict__ Gt,
                                           int tid, float (&acc)[K * K], float& gsum) {
  constexpr int R = K / 2;
  constexpr int TH = kStreamTile, TW = kStreamTileW, HP = kStreamPad, TJ = 4;
  constexpr int AH = TH + 2 * R, AWD = TW + 2 * HP;
  const int r = tid >> 4, c0 = (tid & 15) * TJ;
  WindowStage<TS, 1, AH, AWD, VW> sa;
  WindowStage<TS, 1, TH, TW, VW> sg;
  int b = u_begin / tiles, tile = u_begin - b * tiles;
  auto fetch = [&]() {
    const size_t base = (static_cast<size_t>(b) * C + cc) * plane_stride + sub_off;
    const int ty = tile / tiles_x, tx = tile - ty * tiles_x;
    sa.fetch(A + base, 0, h, w, ty * TH - R, tx * TW - HP, tid);
    sg.fetch(G + base, 0, h, w, ty * TH, tx * TW, tid);
  };
  if (u_begin < u_end) fetch();
  for (int u = u_begin; u < u_end; ++u) {
    sa.commit(At, tid);
    sg.commit(Gt, tid);
    __syncthreads();
    if (++tile == tiles) { tile = 0; ++b; }
    if (u + 1 < u_end) fetch();
    float gv[TJ];
    {
      const float4 t4 = *reinterpret_cast<const float4*>(Gt + r * TW + c0);
      gv[0] = t4.x; gv[1] = t4.y; gv[2] = t4.z; gv[3] = t4.w;
    }
#pragma unroll
    for (int t = 0; t < TJ; ++t) gsum += gv[t];
#pragma unroll
    for (int kh = 0; kh < K; ++kh) {
      float row[12];
      lds_read12(At + (r + kh) * AWD + c0, row);
#pragma unroll
      for (int kw = 0; kw < K; ++kw)
#pragma unroll
        for (int t = 0; t < TJ; ++t)
          acc[kh * K + kw] = fmaf(gv[t], row[t + kw - R + HP], acc[kh * K + kw]);
    }
    __syncthreads();
  }
}

// Correlation sums of one filter set: dWt[kh][kw] = sum_{b,i,j} G[i][j] * A[i+kh-R][j+kw-R].
// The work units are (batch item, tile) pairs, tiles of 16 rows x 64 columns; chunk k of
// gridDim.y takes a contiguous range of them, so that large planes give enough workgroups
// at any batch size.  grid = (C * nsub, nchunk), block = 256; blockIdx.x = c * nsub + s.
// A and G: element type TS, plane (b, c) at plane * plane_stride + s * sub_stride, h x w each.
// A thread owns four adjacent columns (the K rows of A it reads from LDS serve 4 K*K products
// each).  Results: partial[(chunk * C + c) * rec + (f0 + s) * K*K + t], and the plain sum of G
// at partial[... + rec - 1] when `with_gsum` (base conv: the bias gradient).  The partial
// buffer holds `nchunk_total` >= gridDim.y chunk records: a launch with fewer chunks (coarse
// levels with few units) zero-fills its filters in the records it does not use, and chunks
// past the last unit store zeros.  `vec`: rows can be read as 4-element vectors (w % 4 == 0,
// aligned).
template <typename TS, int K>
__global__ __launch_bounds__(256) void stream_corr_kernel(const TS* __restrict__ A, const TS* __restrict__ G,
                                                          size_t plane_stride, size_t sub_stride, int h, int w,
                                                          float* __restrict__ partial, int rec, int f0, int nsub,
                                                          int with_gsum, int B, int C, int vec, int nchunk_total) {
  constexpr int R = K / 2;
  constexpr int TH = kStreamTile, TW = kStreamTileW, HP = kStreamPad;
  constexpr int AH = TH + 2 * R, AWD = TW + 2 * HP;
  constexpr int KK = K * K;
  __shared__ alignas(16) float At[AH * AWD];
  __shared__ alignas(16) float Gt[TH * TW];
  __shared__ float red[4][KK + 1];
  const int cc = blockIdx.x / nsub, s = blockIdx.x - cc * nsub;
  const int chunk = blockIdx.y;
  const int tid = threadIdx.x;
  const int tiles_x = (w + TW - 1) / TW, tiles_y = (h + TH - 1) / TH;
  const int tiles = tiles_x * tiles_y;
  const int units = B * tiles;
  const int per = (units + static_cast<int>(gridDim.y) - 1) / static_cast<int>(gridDim.y);
  const int u_begin = chunk * per;
  const int u_end = u_begin + per < units ? u_begin + per : units;
  float acc[KK];
  float gsum = 0.f;
#pragma unroll
  for (int t = 0; t < KK; ++t) acc[t] = 0.f;
  if (vec) corr_units<TS, K, 4>(A, G, plane_stride, static_cast<size_t>(s) * sub_stride, h, w, C, cc, tiles_x, tiles,
                               u_begin, u_end, At, Gt, tid, acc, gsum);
  else corr_units<TS, K, 1>(A, G, plane_stride, static_cast<size_t>(s) * sub_stride, h, w, C, cc, tiles_x, tiles,
                            u_begin, u_end, At, Gt, tid, acc, gsum);
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
  for (int k = chunk + static_cast<int>(gridDim.y); k < nchunk_total; k += static_cast<int>(gridDim.y)) {
    float* z = partial + (static_cast<size_t>(k) * C + cc) * rec;
    if (tid < KK) z[(f0 + s) * KK + tid] = 0.f;
    if (with_gsum && tid == KK) z[rec - 1] = 0.f;
  }
}

}  // namespace wt
