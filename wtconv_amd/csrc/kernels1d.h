// Tiled WTConv1d kernels for gfx950.
//
// One workgroup owns a tile of T consecutive samples of one (b, c) row plus the halo the
// cascade needs, so rows of any length are handled.  Maths (reference
// wtconv/wtconv1d.py:38-82, wtconv/util/wavelet.py:6-20,46-59):
//   X_0 = x;  A_l = Haar1(zero-pad-to-even(X_{l-1})): lo = (e + o)/sqrt2, hi = (e - o)/sqrt2
//   X_l = A_l[lo];  Y_l[s] = (gamma_l[c,s] w_l[c,s]) (*) A_l[s]   ('same' zero padding)
//   Z_l = crop(iHaar1(Y_l[lo] + Z_{l+1}, Y_l[hi]));  out = gamma_b (w_b (*) x + bias) + Z_1
//
// Halo: the K-tap conv at level l reaches R = K/2 coefficients to each side, and one
// coefficient of level l spans 2 of level l-1, so level l is staged with a halo of
// R * 2^(L-l) coefficients and the input with R * 2^L samples.  Everything outside the
// row is zero, which is at once the 'same' padding of every level and the odd-length
// padding of wtconv1d.py:49-51, because the Haar transform of zeros is zero.
#pragma once

#include "common.h"

namespace wt {

struct Plan1D {
  int C, N, L;
  int T;                       // tile length in samples, multiple of 2^L
  int ntiles;
  int hal[kMaxLevels + 1];     // halo of level l (l = 0: input samples)
  int tl[kMaxLevels + 1];      // tile length at level l: T >> l
  int aoff[kMaxLevels + 1];    // level 0: one buffer; l >= 1: lo then hi
  int apl[kMaxLevels + 1];     // buffer length: tl + 2*hal, rounded up to 4
  int zoff[kMaxLevels + 2];    // Z_l, l = 2..L: tl[l-1] floats
  int goff[kMaxLevels + 1];    // weight-gradient kernel: pyramid of grad_out (no halo,
  int gpl[kMaxLevels + 1];     //   zero padded to the strip width)
  int lds_floats;
  int vec_ok;                  // rows are 16-byte sized and aligned
};

constexpr float kInvSqrt2 = 0.70710678118654752440f;

constexpr int kBlock1D = 256;   // threads per workgroup of the 1-D kernels

// Stage samples [t0 - halo, t0 + T + halo) of one row; zero outside [0, N).
template <typename T>
__device__ __forceinline__ void load_row_tile(const T* __restrict__ row, float* __restrict__ dst,
                                              int N, int start, int count, bool vec) {
  constexpr int EV = 16 / sizeof(T);
  if (vec && (start % EV) == 0) {   // start may be negative: C++ % keeps the test exact for multiples
    const int nv = (count + EV - 1) / EV;
    for (int v = threadIdx.x; v < nv; v += blockDim.x) {
      const int p = start + v * EV;
      float vals[EV];
      if (p >= 0 && p + EV <= N) {
        const uint4 q = *reinterpret_cast<const uint4*>(row + p);
        if constexpr (sizeof(T) == 4) {
          vals[0] = __uint_as_float(q.x); vals[1] = __uint_as_float(q.y);
          vals[2] = __uint_as_float(q.z); vals[3] = __uint_as_float(q.w);
        } else {
          const uint32_t qq[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            unpack2<T>(qq[k], vals[2 * k], vals[2 * k + 1]);
          }
        }
      } else {
#pragma unroll
        for (int k = 0; k < EV; ++k) vals[k] = (p + k >= 0 && p + k < N) ? to_f32<T>(row[p + k]) : 0.f;
      }
#pragma unroll
      for (int k = 0; k < EV; ++k)
        if (v * EV + k < count) dst[v * EV + k] = vals[k];
    }
  } else {
    for (int e = threadIdx.x; e < count; e += blockDim.x) {
      const int p = start + e;
      dst[e] = (p >= 0 && p < N) ? to_f32<T>(row[p]) : 0.f;
    }
  }
}

__device__ __forceinline__ void analysis1d_level(const float* __restrict__ src, float* __restrict__ dst,
                                                 int dpl, int count, int tid, int nthreads) {
  for (int q = tid; q < count; q += nthreads) {
    const float e = src[2 * q], o = src[2 * q + 1];
    dst[q] = (e + o) * kInvSqrt2;
    dst[dpl + q] = (e - o) * kInvSqrt2;
  }
}

template <int K, int TJ>
__device__ __forceinline__ void conv1_strip(const float* __restrict__ a, const float* __restrict__ wf,
                                            float (&y)[TJ]) {
  float row[TJ + K - 1];
#pragma unroll
  for (int q = 0; q < TJ + K - 1; ++q) row[q] = a[q];
#pragma unroll
  for (int k = 0; k < K; ++k) {
    const float wv = wf[k];
#pragma unroll
    for (int t = 0; t < TJ; ++t) y[t] = fmaf(wv, row[t + k], y[t]);
  }
}

template <typename T, int N>
__device__ __forceinline__ void store_run(T* __restrict__ dst, const float (&v)[N], int nvalid, bool vec) {
  if (vec && nvalid == N) {
    if constexpr (sizeof(T) == 4) {
#pragma unroll
      for (int k = 0; k < N / 4; ++k) {
        float4 q;
        q.x = v[4 * k]; q.y = v[4 * k + 1]; q.z = v[4 * k + 2]; q.w = v[4 * k + 3];
        reinterpret_cast<float4*>(dst)[k] = q;
      }
    } else {
#pragma unroll
      for (int k = 0; k < N / 8; ++k) {
        uint4 q;
        q.x = pack2<T>(v[8 * k], v[8 * k + 1]);
        q.y = pack2<T>(v[8 * k + 2], v[8 * k + 3]);
        q.z = pack2<T>(v[8 * k + 4], v[8 * k + 5]);
        q.w = pack2<T>(v[8 * k + 6], v[8 * k + 7]);
        reinterpret_cast<uint4*>(dst)[k] = q;
      }
    }
  } else {
#pragma unroll
    for (int k = 0; k < N; ++k)
      if (k < nvalid) dst[k] = from_f32<T>(v[k]);
  }
}

// Forward / input-gradient kernel.  grid = (ntiles, B*C), block = kBlock1D.
// TJ level-l coefficients (2*TJ outputs of the level below) per work item; TJ = 4.
template <typename T, int K, int TJ>
__global__ __launch_bounds__(kBlock1D) void wt1d_tile_kernel(const T* __restrict__ x, T* __restrict__ out,
                                                        const float* __restrict__ fw,
                                                        const float* __restrict__ fb, Plan1D pl, int nrows) {
  WT_SHARED_FLOATS(lds);
  constexpr int R = K / 2;
  constexpr int NO = 2 * TJ;
  // rows run over gridDim.y and, beyond 65535 of them, gridDim.z (the last z-slice may be ragged)
  const int row = blockIdx.y + blockIdx.z * gridDim.y;
  if (row >= nrows) return;
  const int c = row % pl.C;
  const int t0 = blockIdx.x * pl.T;
  const int NF = 1 + 2 * pl.L;
  const float* fwc = fw + static_cast<size_t>(c) * NF * K;
  const T* xrow = x + static_cast<size_t>(row) * pl.N;
  T* orow = out + static_cast<size_t>(row) * pl.N;

  load_row_tile<T>(xrow, lds + pl.aoff[0], pl.N, t0 - pl.hal[0], pl.tl[0] + 2 * pl.hal[0], pl.vec_ok != 0);
  WT_LDS_BARRIER();
  for (int l = 1; l <= pl.L; ++l) {
    analysis1d_level(lds + pl.aoff[l - 1], lds + pl.aoff[l], pl.apl[l], pl.tl[l] + 2 * pl.hal[l],
                     threadIdx.x, blockDim.x);
    WT_LDS_BARRIER();
  }
  for (int l = pl.L; l >= 2; --l) {
    const int tl = pl.tl[l];
    const int items = (tl + TJ - 1) / TJ;
    const float* A = lds + pl.aoff[l];
    const float* wl_f = fwc + (1 + 2 * (l - 1)) * K;
    const bool has_carry = l < pl.L;
    const float* Zin = lds + pl.zoff[l + 1];
    float* Zout = lds + pl.zoff[l];
    for (int it = threadIdx.x; it < items; it += blockDim.x) {
      const int i0 = it * TJ;
      float lo[TJ], hi[TJ];
#pragma unroll
      for (int t = 0; t < TJ; ++t) { lo[t] = 0.f; hi[t] = 0.f; }
      conv1_strip<K, TJ>(A + i0 + pl.hal[l] - R, wl_f, lo);
      conv1_strip<K, TJ>(A + pl.apl[l] + i0 + pl.hal[l] - R, wl_f + K, hi);
#pragma unroll
      for (int t = 0; t < TJ; ++t) {
        const int i = i0 + t;
        if (i < tl) {
          float v = lo[t];
          if (has_carry) v += Zin[i];
          Zout[2 * i] = (v + hi[t]) * kInvSqrt2;
          Zout[2 * i + 1] = (v - hi[t]) * kInvSqrt2;
        }
      }
    }
    WT_LDS_BARRIER();
  }
  {
    const int tl = pl.tl[1];
    const int items = (tl + TJ - 1) / TJ;
    const float* A = lds + pl.aoff[1];
    const float* X = lds + pl.aoff[0];
    const float* w1_f = fwc + K;
    const bool has_carry = pl.L > 1;
    const float* Zin = lds + pl.zoff[2];
    const float bias = fb[c];
    const bool vec = pl.vec_ok != 0;
    for (int it = threadIdx.x; it < items; it += blockDim.x) {
      const int i0 = it * TJ;
      float lo[TJ], hi[TJ];
#pragma unroll
      for (int t = 0; t < TJ; ++t) { lo[t] = 0.f; hi[t] = 0.f; }
      conv1_strip<K, TJ>(A + i0 + pl.hal[1] - R, w1_f, lo);
      conv1_strip<K, TJ>(A + pl.apl[1] + i0 + pl.hal[1] - R, w1_f + K, hi);
      float o[NO];
#pragma unroll
      for (int t = 0; t < NO; ++t) o[t] = bias;
      conv1_strip<K, NO>(X + 2 * i0 + pl.hal[0] - R, fwc, o);
#pragma unroll
      for (int t = 0; t < TJ; ++t) {
        float v = lo[t];
        if (has_carry && i0 + t < tl) v += Zin[i0 + t];
        o[2 * t] += (v + hi[t]) * kInvSqrt2;
        o[2 * t + 1] += (v - hi[t]) * kInvSqrt2;
      }
      const int p = t0 + 2 * i0;
      int nvalid = pl.N - p;
      const int in_tile = 2 * (tl - i0);
      if (nvalid > in_tile) nvalid = in_tile;
      if (nvalid > NO) nvalid = NO;
      if (nvalid > 0) store_run<T, NO>(orow + p, o, nvalid, vec);
    }
  }
}

// Parameter gradients, first stage.  grid = (C, nchunk), block = kBlock1D.  A workgroup walks
// `per_chunk` (row, tile) pairs of one channel, every thread keeps K sums per filter in
// registers; reduction and output layout as in the 2-D kernel:
//   partial[chunk][c][ (1 + 2L) * K + 1 ]
template <int K, int TJ>
__device__ __forceinline__ void corr1_strip(const float* __restrict__ a, const float* __restrict__ gy,
                                            float (&acc)[K]) {
  float row[TJ + K - 1];
#pragma unroll
  for (int q = 0; q < TJ + K - 1; ++q) row[q] = a[q];
#pragma unroll
  for (int t = 0; t < TJ; ++t) {
    const float dy = gy[t];
#pragma unroll
    for (int k = 0; k < K; ++k) acc[k] = fmaf(dy, row[t + k], acc[k]);
  }
}

template <typename T, int K, int L, int TJ>
__global__ __launch_bounds__(kBlock1D) void wt1d_wgrad_kernel(const T* __restrict__ x, const T* __restrict__ g,
                                                         float* __restrict__ partial, Plan1D pl, int B,
                                                         int per_chunk) {
  WT_SHARED_FLOATS(lds);
  constexpr int R = K / 2;
  constexpr int NF = 1 + 2 * L;
  const int c = blockIdx.x;
  const int chunk = blockIdx.y;
  const int tid = threadIdx.x;

  float accb[K];
  float accl[L][2][K];
  float gsum = 0.f;
#pragma unroll
  for (int k = 0; k < K; ++k) accb[k] = 0.f;
#pragma unroll
  for (int l = 0; l < L; ++l)
#pragma unroll
    for (int k = 0; k < K; ++k) { accl[l][0][k] = 0.f; accl[l][1][k] = 0.f; }

  for (int v = tid; v < pl.lds_floats; v += blockDim.x) lds[v] = 0.f;
  WT_LDS_BARRIER();

  const int total = B * pl.ntiles;
  const int w_end = (chunk + 1) * per_chunk < total ? (chunk + 1) * per_chunk : total;
  for (int wi = chunk * per_chunk; wi < w_end; ++wi) {
    const int b = wi / pl.ntiles;
    const int t0 = (wi - b * pl.ntiles) * pl.T;
    const size_t roff = (static_cast<size_t>(b) * pl.C + c) * pl.N;
    load_row_tile<T>(x + roff, lds + pl.aoff[0], pl.N, t0 - pl.hal[0], pl.tl[0] + 2 * pl.hal[0], pl.vec_ok != 0);
    load_row_tile<T>(g + roff, lds + pl.goff[0], pl.N, t0, pl.tl[0], pl.vec_ok != 0);
    WT_LDS_BARRIER();
#pragma unroll
    for (int l = 1; l <= L; ++l) {
      analysis1d_level(lds + pl.aoff[l - 1], lds + pl.aoff[l], pl.apl[l], pl.tl[l] + 2 * pl.hal[l], tid, blockDim.x);
      analysis1d_level(lds + pl.goff[l - 1], lds + pl.goff[l], pl.gpl[l], pl.tl[l], tid, blockDim.x);
      WT_LDS_BARRIER();
    }
    {
      const int items = (pl.tl[0] + TJ - 1) / TJ;
      const float* X = lds + pl.aoff[0];
      const float* G = lds + pl.goff[0];
      for (int it = tid; it < items; it += blockDim.x) {
        const int i0 = it * TJ;
#pragma unroll
        for (int t = 0; t < TJ; ++t) gsum += G[i0 + t];
        corr1_strip<K, TJ>(X + i0 + pl.hal[0] - R, G + i0, accb);
      }
    }
#pragma unroll
    for (int l = 1; l <= L; ++l) {
      const int items = (pl.tl[l] + TJ - 1) / TJ;
      const float* A = lds + pl.aoff[l];
      const float* G = lds + pl.goff[l];
      for (int it = tid; it < items; it += blockDim.x) {
        const int i0 = it * TJ;
        corr1_strip<K, TJ>(A + i0 + pl.hal[l] - R, G + i0, accl[l - 1][0]);
        corr1_strip<K, TJ>(A + pl.apl[l] + i0 + pl.hal[l] - R, G + pl.gpl[l] + i0, accl[l - 1][1]);
      }
    }
    WT_LDS_BARRIER();
  }

  constexpr int NRED = NF * K + 1;
  float* red = lds;   // [waves][NRED]
  const int wave = tid >> 6, lane = tid & (kWave - 1);
#pragma unroll
  for (int k = 0; k < K; ++k) {
    const float v = wave_sum(accb[k]);
    if (lane == 0) red[wave * NRED + k] = v;
  }
#pragma unroll
  for (int l = 0; l < L; ++l)
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int k = 0; k < K; ++k) {
        const float v = wave_sum(accl[l][s][k]);
        if (lane == 0) red[wave * NRED + (1 + 2 * l + s) * K + k] = v;
      }
  {
    const float v = wave_sum(gsum);
    if (lane == 0) red[wave * NRED + NRED - 1] = v;
  }
  WT_LDS_BARRIER();
  float* dst = partial + (static_cast<size_t>(chunk) * pl.C + c) * NRED;
  const int nwaves = blockDim.x >> 6;
  for (int o = tid; o < NRED; o += blockDim.x) {
    float v = 0.f;
    for (int wv = 0; wv < nwaves; ++wv) v += red[wv * NRED + o];
    dst[o] = v;
  }
}

}  // namespace wt
