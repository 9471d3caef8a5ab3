// Single-level Haar (db1) transforms as operators of their own: what wtconv/util/wavelet.py:46-75 of the reference
// computes with a stride-2 grouped convolution against the db1 filter bank (analysis) and the matching transposed
// convolution (synthesis), for even extents.  Sub-band order as in the bank (wavelet.py:26-29): LL, LH, HL, HH with
//   LL = (a + b + c + d) / 2, LH = (a + b - c - d) / 2, HL = (a - b + c - d) / 2, HH = (a - b - c + d) / 2
// for the 2 x 2 block [[a, b], [c, d]]; 1-D: lo = (e + o) / sqrt 2, hi = (e - o) / sqrt 2.  The transforms are
// orthogonal, so each is the other's adjoint (which is all their autograd needs).  Pure streaming kernels: a thread
// moves two adjacent coefficient positions (four input columns) per row pair.
#pragma once

#include "common.h"

namespace wt {

constexpr int kHaarThreads = 256;

// x (planes, H, W) -> out (planes, 4, H/2, W/2).  Grid (ceil(h * ceil(w / 2) / 256), planes folded into y and z).
template <typename T>
__global__ void __launch_bounds__(kHaarThreads)
haar2d_analysis_kernel(const T* __restrict__ x, T* __restrict__ out, int h, int w, long long planes) {
  const long long plane = static_cast<long long>(blockIdx.z) * gridDim.y + blockIdx.y;
  if (plane >= planes) return;
  const int wp = (w + 1) >> 1;                       // pairs of coefficient columns per row
  const int item = blockIdx.x * kHaarThreads + threadIdx.x;
  if (item >= h * wp) return;
  const int i = item / wp, jp = item - i * wp, j = 2 * jp;
  const int W = 2 * w;
  const T* src = x + plane * (4LL * h * w) + static_cast<long long>(2 * i) * W + 2 * j;
  T* dst = out + plane * (4LL * h * w) + static_cast<long long>(i) * w + j;
  const long long sub = static_cast<long long>(h) * w;
  const int n = j + 1 < w ? 2 : 1;
  for (int k = 0; k < n; ++k) {
    const float a = to_f32<T>(src[2 * k]), b = to_f32<T>(src[2 * k + 1]);
    const float c = to_f32<T>(src[W + 2 * k]), d = to_f32<T>(src[W + 2 * k + 1]);
    const float s1 = a + b, d1 = a - b, s2 = c + d, d2 = c - d;
    dst[k] = from_f32<T>(0.5f * (s1 + s2));
    dst[sub + k] = from_f32<T>(0.5f * (s1 - s2));
    dst[2 * sub + k] = from_f32<T>(0.5f * (d1 + d2));
    dst[3 * sub + k] = from_f32<T>(0.5f * (d1 - d2));
  }
}

// coef (planes, 4, h, w) -> out (planes, 2h, 2w)
template <typename T>
__global__ void __launch_bounds__(kHaarThreads)
haar2d_synthesis_kernel(const T* __restrict__ coef, T* __restrict__ out, int h, int w, long long planes) {
  const long long plane = static_cast<long long>(blockIdx.z) * gridDim.y + blockIdx.y;
  if (plane >= planes) return;
  const int wp = (w + 1) >> 1;
  const int item = blockIdx.x * kHaarThreads + threadIdx.x;
  if (item >= h * wp) return;
  const int i = item / wp, jp = item - i * wp, j = 2 * jp;
  const int W = 2 * w;
  const long long sub = static_cast<long long>(h) * w;
  const T* src = coef + plane * (4LL * h * w) + static_cast<long long>(i) * w + j;
  T* dst = out + plane * (4LL * h * w) + static_cast<long long>(2 * i) * W + 2 * j;
  const int n = j + 1 < w ? 2 : 1;
  for (int k = 0; k < n; ++k) {
    const float ll = to_f32<T>(src[k]), lh = to_f32<T>(src[sub + k]);
    const float hl = to_f32<T>(src[2 * sub + k]), hh = to_f32<T>(src[3 * sub + k]);
    const float p = ll + lh, m = ll - lh, q = hl + hh, r = hl - hh;
    dst[2 * k] = from_f32<T>(0.5f * (p + q));
    dst[2 * k + 1] = from_f32<T>(0.5f * (p - q));
    dst[W + 2 * k] = from_f32<T>(0.5f * (m + r));
    dst[W + 2 * k + 1] = from_f32<T>(0.5f * (m - r));
  }
}

// x (rows, N) -> out (rows, 2, N/2); inverse != 0: coef (rows, 2, n) -> out (rows, 2n).  Grid (ceil(n / 256), rows
// folded into y and z).
template <typename T>
__global__ void __launch_bounds__(kHaarThreads)
haar1d_kernel(const T* __restrict__ x, T* __restrict__ out, int n, long long rows, int inverse) {
  const long long row = static_cast<long long>(blockIdx.z) * gridDim.y + blockIdx.y;
  if (row >= rows) return;
  const int q = blockIdx.x * kHaarThreads + threadIdx.x;
  if (q >= n) return;
  constexpr float kR = 0.70710678118654752440f;
  const T* src = x + row * (2LL * n);
  T* dst = out + row * (2LL * n);
  if (!inverse) {
    const float e = to_f32<T>(src[2 * q]), o = to_f32<T>(src[2 * q + 1]);
    dst[q] = from_f32<T>((e + o) * kR);
    dst[n + q] = from_f32<T>((e - o) * kR);
  } else {
    const float lo = to_f32<T>(src[q]), hi = to_f32<T>(src[n + q]);
    dst[2 * q] = from_f32<T>((lo + hi) * kR);
    dst[2 * q + 1] = from_f32<T>((lo - hi) * kR);
  }
}

}  // namespace wt
