// Plane-resident WTConv2d kernels for gfx950.
//
// One workgroup owns one (b, c) plane.  The plane, the Haar pyramid built from it and
// the partial reconstructions all live in LDS, so HBM sees the plane once on the way in
// and the result once on the way out.
//
// Maths (reference wtconv/wtconv2d.py:38-82; sub-band convention
// fast_wtconv/cuda_haar/haar_common.cuh:4-15):
//   X_0 = x;  A_l = Haar(zero-pad-to-even(X_{l-1}));  X_l = A_l[LL]
//   Y_l[s] = (gamma_l[c,s] * w_l[c,s]) (*) A_l[s]          'same' zero padding
//   Z_{L+1} = 0;  Z_l = crop(iHaar(Y_l[LL] + Z_{l+1}, Y_l[LH], Y_l[HL], Y_l[HH]))
//   out = gamma_b[c] * (w_b[c] (*) x + bias[c]) + Z_1
// The bias-free part is linear and its adjoint has the same structure with every kernel
// rotated by 180 degrees, so the same kernel run on grad_out with flipped folded weights
// yields grad_x.
#pragma once

#include "common.h"

namespace wt {

// LDS layout of one plane, computed on the host (plan.h).
struct Plan2D {
  int C, H, W, L;
  int P;                       // halo width of the pyramid buffers: max(K/2, 1)
  int h[kMaxLevels + 1];       // grid of level l (l = 0 is the input plane)
  int w[kMaxLevels + 1];
  int aoff[kMaxLevels + 1];    // float offset of level l (level 0: 1 plane; l >= 1: 4 planes)
  int astr[kMaxLevels + 1];    // row stride
  int apl[kMaxLevels + 1];     // size of one sub-band plane
  int zoff[kMaxLevels + 2];    // Z_l for l = 2..L, shape h[l-1] x w[l-1]
  int zstr[kMaxLevels + 2];
  int goff[kMaxLevels + 1];    // weight-gradient kernel only: pyramid of grad_out,
  int gstr[kMaxLevels + 1];    //   zero padded on the right/bottom, no halo
  int gpl[kMaxLevels + 1];
  int lds_floats;              // total, including slack
  int vec_ok;                  // planes are 16-byte sized and aligned: 128-bit loads
  int row_vec_ok;              // output row pieces may be stored as vectors
};

// ------------------------------------------------------------------ parameter folding
// fw[c][f][t]: f = 0 base conv, f = 1 + S*l + s level l sub-band s; value gamma * w, taps
// reversed when flip != 0.  fb[c] = gamma_b * bias (0 without bias).
__global__ void fold_params_kernel(ParamTable p, int pdtype, float* __restrict__ fw,
                                   float* __restrict__ fb, int C, int S, int L, int KK,
                                   int flip, int use_bias) {
  const int NF = 1 + S * L;
  const int total = C * NF * KK;
  for (int idx = blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += gridDim.x * blockDim.x) {
    const int t = idx % KK;
    const int f = (idx / KK) % NF;
    const int c = idx / (KK * NF);
    const int ts = flip ? KK - 1 - t : t;
    float v;
    if (f == 0) {
      v = load_param(p.base_weight, pdtype, c * KK + ts) * load_param(p.base_scale, pdtype, c);
    } else {
      const int l = (f - 1) / S, s = (f - 1) % S;
      const int ch = c * S + s;
      v = load_param(p.wt_weight[l], pdtype, ch * KK + ts) * load_param(p.wt_scale[l], pdtype, ch);
    }
    fw[idx] = v;
    if (f == 0 && t == 0) {
      fb[c] = (use_bias && p.base_bias != nullptr)
                  ? load_param(p.base_bias, pdtype, c) * load_param(p.base_scale, pdtype, c)
                  : 0.f;
    }
  }
}

// ------------------------------------------------------------------ plane load
// Copy one contiguous H x W plane from HBM into a haloed (or padded) LDS buffer whose
// element (r, col) sits at dst[(r + P) * str + col + P].
template <typename T>
__device__ __forceinline__ void load_plane(const T* __restrict__ src, float* __restrict__ dst,
                                           int H, int W, int str, int P, bool vec) {
  const int n = H * W;
  if (vec) {
    constexpr int EV = 16 / sizeof(T);
    const int nv = n / EV;
    const uint4* __restrict__ s4 = reinterpret_cast<const uint4*>(src);
    for (int v = threadIdx.x; v < nv; v += blockDim.x) {
      const uint4 q = s4[v];
      float vals[EV];
      if constexpr (sizeof(T) == 4) {
        vals[0] = __uint_as_float(q.x); vals[1] = __uint_as_float(q.y);
        vals[2] = __uint_as_float(q.z); vals[3] = __uint_as_float(q.w);
      } else {
        const uint32_t qq[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          vals[2 * k] = __uint_as_float(qq[k] << 16);
          vals[2 * k + 1] = __uint_as_float(qq[k] & 0xffff0000u);
        }
      }
      const int e = v * EV;
      int r = e / W;
      int col = e - r * W;
#pragma unroll
      for (int k = 0; k < EV; ++k) {
        dst[(r + P) * str + col + P] = vals[k];
        if (++col == W) { col = 0; ++r; }
      }
    }
  } else {
    for (int e = threadIdx.x; e < n; e += blockDim.x) {
      const int r = e / W, col = e - r * W;
      dst[(r + P) * str + col + P] = to_f32<T>(src[e]);
    }
  }
}

// One analysis level: src is the (haloed/padded, zero outside) LL plane of level l-1,
// dst the four sub-band planes of level l.  Reading one past the source grid returns the
// zero padding the reference applies to odd sizes (wtconv2d.py:49-51).
__device__ __forceinline__ void analysis_level(const float* __restrict__ src, int sstr, int sP,
                                               float* __restrict__ dst, int dstr, int dpl, int dP,
                                               int hl, int wl, int tid, int nthreads) {
  const int items = hl * wl;
  for (int it = tid; it < items; it += nthreads) {
    const int i = it / wl, j = it - i * wl;
    const float* s0 = src + (2 * i + sP) * sstr + 2 * j + sP;
    const float a = s0[0], b = s0[1], c = s0[sstr], d = s0[sstr + 1];
    const float sac = a + c, sbd = b + d, dac = a - c, dbd = b - d;
    float* o = dst + (i + dP) * dstr + j + dP;
    o[0] = 0.5f * (sac + sbd);
    o[dpl] = 0.5f * (dac + dbd);
    o[2 * dpl] = 0.5f * (sac - sbd);
    o[3 * dpl] = 0.5f * (dac - dbd);
  }
}

// Load NR consecutive floats from LDS as vectors of VW floats (VW = 4: ds_read_b128,
// VW = 2: ds_read_b64).  The address must be VW*4-byte aligned.
template <int NR, int VW>
__device__ __forceinline__ void lds_row(const float* __restrict__ a, float (&row)[NR]) {
  static_assert(NR % VW == 0, "row length is padded to the vector width");
  if constexpr (VW == 4) {
#pragma unroll
    for (int q = 0; q < NR / 4; ++q) {
      const float4 v = reinterpret_cast<const float4*>(a)[q];
      row[4 * q] = v.x; row[4 * q + 1] = v.y; row[4 * q + 2] = v.z; row[4 * q + 3] = v.w;
    }
  } else if constexpr (VW == 2) {
#pragma unroll
    for (int q = 0; q < NR / 2; ++q) {
      const float2 v = reinterpret_cast<const float2*>(a)[q];
      row[2 * q] = v.x; row[2 * q + 1] = v.y;
    }
  } else {
#pragma unroll
    for (int q = 0; q < NR; ++q) row[q] = a[q];
  }
}

constexpr int pad_to(int n, int m) { return (n + m - 1) / m * m; }

// K x K correlation of TJ horizontally adjacent outputs; `a` points at the top-left input
// of the first output's window (VW*4-byte aligned).
template <int K, int TJ, int VW>
__device__ __forceinline__ void conv_strip(const float* __restrict__ a, int astr,
                                           const float* __restrict__ wf, float (&y)[TJ]) {
  constexpr int NR = pad_to(TJ + K - 1, VW);
#pragma unroll
  for (int kh = 0; kh < K; ++kh) {
    float row[NR];
    lds_row<NR, VW>(a + kh * astr, row);
#pragma unroll
    for (int kw = 0; kw < K; ++kw) {
      const float wv = wf[kh * K + kw];
#pragma unroll
      for (int t = 0; t < TJ; ++t) y[t] = fmaf(wv, row[t + kw], y[t]);
    }
  }
}

__device__ __forceinline__ void ihaar4(float ll, float lh, float hl, float hh,
                                       float& a, float& b, float& c, float& d) {
  const float p = ll + lh, m = ll - lh, q = hl + hh, n = hl - hh;
  a = 0.5f * (p + q);
  b = 0.5f * (p - q);
  c = 0.5f * (m + n);
  d = 0.5f * (m - n);
}

// Synthesis of an inner level l (2 <= l <= L): conv of the four sub-bands, add Z_{l+1},
// inverse Haar, cropped store into Z_l.
template <int K, int TJ>
__device__ __forceinline__ void synth_inner(float* __restrict__ lds, const Plan2D& pl, int l,
                                            const float* __restrict__ wl_f) {
  constexpr int R = K / 2;
  constexpr int VW = (R >= 1) ? TJ : 1;   // window starts at column j0 when the halo equals R
  const int hl = pl.h[l], wl = pl.w[l];
  const int nstrip = (wl + TJ - 1) / TJ;
  const int items = hl * nstrip;
  const int astr = pl.astr[l], apl = pl.apl[l], P = pl.P;
  const float* A = lds + pl.aoff[l];
  const bool has_carry = l < pl.L;
  const float* Zin = lds + pl.zoff[l + 1];
  const int zin_str = pl.zstr[l + 1];
  float* Zout = lds + pl.zoff[l];
  const int zout_str = pl.zstr[l];
  const int ho = pl.h[l - 1], wo = pl.w[l - 1];
  for (int it = threadIdx.x; it < items; it += blockDim.x) {
    const int i = it / nstrip;
    const int j0 = (it - i * nstrip) * TJ;
    float y[4][TJ];
#pragma unroll
    for (int s = 0; s < 4; ++s) {
#pragma unroll
      for (int t = 0; t < TJ; ++t) y[s][t] = 0.f;
      conv_strip<K, TJ, VW>(A + s * apl + (i - R + P) * astr + (j0 - R + P), astr, wl_f + s * K * K, y[s]);
    }
#pragma unroll
    for (int t = 0; t < TJ; ++t) {
      const int j = j0 + t;
      float ll = y[0][t];
      if (has_carry) ll += Zin[i * zin_str + j];
      float a, b, c, d;
      ihaar4(ll, y[1][t], y[2][t], y[3][t], a, b, c, d);
      const int r0 = 2 * i, c0 = 2 * j;
      if (j < wl) {
        if (c0 < wo) {
          Zout[r0 * zout_str + c0] = a;
          if (r0 + 1 < ho) Zout[(r0 + 1) * zout_str + c0] = c;
        }
        if (c0 + 1 < wo) {
          Zout[r0 * zout_str + c0 + 1] = b;
          if (r0 + 1 < ho) Zout[(r0 + 1) * zout_str + c0 + 1] = d;
        }
      }
    }
  }
}

template <typename T, int N>
__device__ __forceinline__ void store_row(T* __restrict__ dst, const float (&v)[N], int nvalid, bool vec) {
  if (vec && nvalid == N) {
    if constexpr (sizeof(T) == 4) {
      static_assert(N % 4 == 0, "row pieces are multiples of 4 elements");
#pragma unroll
      for (int k = 0; k < N / 4; ++k) {
        float4 q;
        q.x = v[4 * k]; q.y = v[4 * k + 1]; q.z = v[4 * k + 2]; q.w = v[4 * k + 3];
        reinterpret_cast<float4*>(dst)[k] = q;
      }
    } else {
      static_assert(N % 4 == 0, "row pieces are multiples of 4 elements");
#pragma unroll
      for (int k = 0; k < N / 4; ++k) {
        uint2 q;
        q.x = static_cast<uint32_t>(f32_to_bf16(v[4 * k])) | (static_cast<uint32_t>(f32_to_bf16(v[4 * k + 1])) << 16);
        q.y = static_cast<uint32_t>(f32_to_bf16(v[4 * k + 2])) | (static_cast<uint32_t>(f32_to_bf16(v[4 * k + 3])) << 16);
        reinterpret_cast<uint2*>(dst)[k] = q;
      }
    }
  } else {
#pragma unroll
    for (int k = 0; k < N; ++k)
      if (k < nvalid) dst[k] = from_f32<T>(v[k]);
  }
}

// Level 1: conv of the four sub-bands, add Z_2, inverse Haar, add the scaled base conv
// (and bias) of the same 2 x 2TJ pixels, store to HBM.
template <typename T, int K, int TJ>
__device__ __forceinline__ void synth_final(float* __restrict__ lds, const Plan2D& pl,
                                            const float* __restrict__ wb_f,
                                            const float* __restrict__ w1_f, float bias,
                                            T* __restrict__ out_plane) {
  constexpr int R = K / 2;
  constexpr int NO = 2 * TJ;
  constexpr int VW = (R >= 1) ? TJ : 1;
  constexpr int VWX = (R >= 1) ? (NO >= 4 ? 4 : NO) : 1;
  const int hl = pl.h[1], wl = pl.w[1];
  const int nstrip = (wl + TJ - 1) / TJ;
  const int items = hl * nstrip;
  const int astr = pl.astr[1], apl = pl.apl[1], P = pl.P;
  const float* A = lds + pl.aoff[1];
  const float* X = lds + pl.aoff[0];
  const int xstr = pl.astr[0];
  const bool has_carry = pl.L > 1;
  const float* Zin = lds + pl.zoff[2];
  const int zin_str = pl.zstr[2];
  const int H = pl.H, W = pl.W;
  for (int it = threadIdx.x; it < items; it += blockDim.x) {
    const int i = it / nstrip;
    const int j0 = (it - i * nstrip) * TJ;
    float y[4][TJ];
#pragma unroll
    for (int s = 0; s < 4; ++s) {
#pragma unroll
      for (int t = 0; t < TJ; ++t) y[s][t] = 0.f;
      conv_strip<K, TJ, VW>(A + s * apl + (i - R + P) * astr + (j0 - R + P), astr, w1_f + s * K * K, y[s]);
    }
    float o0[NO], o1[NO];
#pragma unroll
    for (int t = 0; t < TJ; ++t) {
      float ll = y[0][t];
      if (has_carry) ll += Zin[i * zin_str + j0 + t];
      ihaar4(ll, y[1][t], y[2][t], y[3][t], o0[2 * t], o0[2 * t + 1], o1[2 * t], o1[2 * t + 1]);
    }
    // base conv of output rows 2i, 2i+1, columns 2j0 .. 2j0+NO-1
    float b0[NO], b1[NO];
#pragma unroll
    for (int t = 0; t < NO; ++t) { b0[t] = bias; b1[t] = bias; }
    const float* xw = X + (2 * i - R + P) * xstr + (2 * j0 - R + P);
#pragma unroll
    for (int r = 0; r < K + 1; ++r) {
      constexpr int NRX = pad_to(NO + K - 1, VWX);
      float row[NRX];
      lds_row<NRX, VWX>(xw + r * xstr, row);
      if (r < K) {
#pragma unroll
        for (int kw = 0; kw < K; ++kw) {
          const float wv = wb_f[r * K + kw];
#pragma unroll
          for (int t = 0; t < NO; ++t) b0[t] = fmaf(wv, row[t + kw], b0[t]);
        }
      }
      if (r >= 1) {
#pragma unroll
        for (int kw = 0; kw < K; ++kw) {
          const float wv = wb_f[(r - 1) * K + kw];
#pragma unroll
          for (int t = 0; t < NO; ++t) b1[t] = fmaf(wv, row[t + kw], b1[t]);
        }
      }
    }
#pragma unroll
    for (int t = 0; t < NO; ++t) { o0[t] += b0[t]; o1[t] += b1[t]; }
    const int r0 = 2 * i, c0 = 2 * j0;
    int nvalid = W - c0;
    if (nvalid > NO) nvalid = NO;
    if (nvalid > 0) {
      store_row<T, NO>(out_plane + r0 * W + c0, o0, nvalid, pl.row_vec_ok != 0);
      if (r0 + 1 < H) store_row<T, NO>(out_plane + (r0 + 1) * W + c0, o1, nvalid, pl.row_vec_ok != 0);
    }
  }
}

__device__ __forceinline__ void zero_lds(float* lds, int nfloats) {
  // nfloats is a multiple of 4 (plan.h) and the buffer is 16-byte aligned
  float4 z;
  z.x = z.y = z.z = z.w = 0.f;
  float4* p = reinterpret_cast<float4*>(lds);
  for (int v = threadIdx.x; v < nfloats / 4; v += blockDim.x) p[v] = z;
}

// Forward (and, with flipped folded weights and zero fb, input-gradient) kernel.
// grid.x = B*C planes, block = 256 threads.
template <typename T, int K, int TJ1, int TJC>
__global__ __launch_bounds__(256) void wt2d_plane_kernel(const T* __restrict__ x, T* __restrict__ out,
                                                         const float* __restrict__ fw,
                                                         const float* __restrict__ fb, Plan2D pl) {
  WT_SHARED_FLOATS(lds);
  constexpr int KK = K * K;
  const int plane = blockIdx.x;
  const int c = plane % pl.C;
  const int NF = 1 + 4 * pl.L;
  const float* fwc = fw + static_cast<size_t>(c) * NF * KK;
  const size_t plane_off = static_cast<size_t>(plane) * pl.H * pl.W;

  zero_lds(lds, pl.lds_floats);
  __syncthreads();
  load_plane<T>(x + plane_off, lds + pl.aoff[0], pl.H, pl.W, pl.astr[0], pl.P, pl.vec_ok != 0);
  __syncthreads();
  for (int l = 1; l <= pl.L; ++l) {
    const float* src = lds + pl.aoff[l - 1];   // sub-band 0 (or the input plane)
    analysis_level(src, pl.astr[l - 1], pl.P, lds + pl.aoff[l], pl.astr[l], pl.apl[l], pl.P,
                   pl.h[l], pl.w[l], threadIdx.x, blockDim.x);
    __syncthreads();
  }
  for (int l = pl.L; l >= 2; --l) {
    synth_inner<K, TJC>(lds, pl, l, fwc + (1 + 4 * (l - 1)) * KK);
    __syncthreads();
  }
  synth_final<T, K, TJ1>(lds, pl, fwc, fwc + KK, fb[c], out + plane_off);
}

// ------------------------------------------------------------------ parameter gradients
// grid = (C, nchunk), block = 512 threads = 8 waves.  Each workgroup walks `bchunk`
// planes of one channel; wave w accumulates, in registers, the K*K correlation sums of
// sub-band (w & 3) at every level plus its share of the base-conv sums.  One cross-lane
// reduction at the end, partial sums to HBM, finished by wgrad_finish_kernel (two-stage,
// deterministic; the reference uses float atomics, fused_haar_conv.cu:331-341).
//   dWt_l[c,s,kh,kw] = sum_{b,i,j} dY_l[s][i,j] * A_l[s][i+kh-R, j+kw-R]
//   dWt_b[c,kh,kw]   = sum_{b,i,j} G[i,j] * x[i+kh-R, j+kw-R],   sumG[c] = sum G
template <int K, int TJ, int VW>
__device__ __forceinline__ void corr_strip(const float* __restrict__ a, int astr,
                                           const float* __restrict__ gy, float (&acc)[K * K]) {
  constexpr int NR = pad_to(TJ + K - 1, VW);
  float dy[TJ];
  lds_row<TJ, (TJ % 4 == 0) ? 4 : 1>(gy, dy);
#pragma unroll
  for (int kh = 0; kh < K; ++kh) {
    float row[NR];
    lds_row<NR, VW>(a + kh * astr, row);
#pragma unroll
    for (int kw = 0; kw < K; ++kw) {
#pragma unroll
      for (int t = 0; t < TJ; ++t) acc[kh * K + kw] = fmaf(dy[t], row[t + kw], acc[kh * K + kw]);
    }
  }
}

template <typename T, int K, int L, int TJ>
__global__ __launch_bounds__(512) void wt2d_wgrad_kernel(const T* __restrict__ x, const T* __restrict__ g,
                                                         float* __restrict__ partial, Plan2D pl,
                                                         int B, int bchunk) {
  WT_SHARED_FLOATS(lds);
  constexpr int KK = K * K;
  constexpr int R = K / 2;
  constexpr int NF = 1 + 4 * L;
  constexpr int VW = (R >= 1 && TJ % 4 == 0) ? 4 : 1;
  const int c = blockIdx.x;
  const int chunk = blockIdx.y;
  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int sb = wave & 3;
  const int sub_tid = (wave >> 2) * kWave + (tid & (kWave - 1));   // 0..127 within the sub-band group
  const int P = pl.P;

  float accb[KK];
  float accl[L][KK];
  float gsum = 0.f;
#pragma unroll
  for (int t = 0; t < KK; ++t) accb[t] = 0.f;
#pragma unroll
  for (int l = 0; l < L; ++l)
#pragma unroll
    for (int t = 0; t < KK; ++t) accl[l][t] = 0.f;

  zero_lds(lds, pl.lds_floats);
  __syncthreads();

  const int b_end = (chunk + 1) * bchunk < B ? (chunk + 1) * bchunk : B;
  for (int b = chunk * bchunk; b < b_end; ++b) {
    const size_t plane_off = (static_cast<size_t>(b) * pl.C + c) * pl.H * pl.W;
    load_plane<T>(x + plane_off, lds + pl.aoff[0], pl.H, pl.W, pl.astr[0], P, pl.vec_ok != 0);
    load_plane<T>(g + plane_off, lds + pl.goff[0], pl.H, pl.W, pl.gstr[0], 0, pl.vec_ok != 0);
    __syncthreads();
#pragma unroll
    for (int l = 1; l <= L; ++l) {
      analysis_level(lds + pl.aoff[l - 1], pl.astr[l - 1], P, lds + pl.aoff[l], pl.astr[l], pl.apl[l], P,
                     pl.h[l], pl.w[l], tid, blockDim.x);
      analysis_level(lds + pl.goff[l - 1], pl.gstr[l - 1], 0, lds + pl.goff[l], pl.gstr[l], pl.gpl[l], 0,
                     pl.h[l], pl.w[l], tid, blockDim.x);
      __syncthreads();
    }
    {  // base conv: all threads share the full-resolution plane
      const int nstrip = (pl.W + TJ - 1) / TJ;
      const int items = pl.H * nstrip;
      const float* X = lds + pl.aoff[0];
      const float* G = lds + pl.goff[0];
      for (int it = tid; it < items; it += blockDim.x) {
        const int i = it / nstrip;
        const int j0 = (it - i * nstrip) * TJ;
        const float* gy = G + i * pl.gstr[0] + j0;
#pragma unroll
        for (int t = 0; t < TJ; ++t) gsum += gy[t];
        corr_strip<K, TJ, VW>(X + (i - R + P) * pl.astr[0] + (j0 - R + P), pl.astr[0], gy, accb);
      }
    }
#pragma unroll
    for (int l = 1; l <= L; ++l) {
      const int nstrip = (pl.w[l] + TJ - 1) / TJ;
      const int items = pl.h[l] * nstrip;
      const float* A = lds + pl.aoff[l] + sb * pl.apl[l];
      const float* G = lds + pl.goff[l] + sb * pl.gpl[l];
      for (int it = sub_tid; it < items; it += 2 * kWave) {
        const int i = it / nstrip;
        const int j0 = (it - i * nstrip) * TJ;
        corr_strip<K, TJ, VW>(A + (i - R + P) * pl.astr[l] + (j0 - R + P), pl.astr[l],
                          G + i * pl.gstr[l] + j0, accl[l - 1]);
      }
    }
    __syncthreads();
  }

  // cross-lane reduction, then cross-wave through LDS (pyramid buffers are dead now)
  constexpr int NRED = KK * (L + 1) + 1;
  float* red = lds;   // [8 waves][NRED]
  const int lane = tid & (kWave - 1);
#pragma unroll
  for (int t = 0; t < KK; ++t) {
    const float v = wave_sum(accb[t]);
    if (lane == 0) red[wave * NRED + t] = v;
  }
#pragma unroll
  for (int l = 0; l < L; ++l)
#pragma unroll
    for (int t = 0; t < KK; ++t) {
      const float v = wave_sum(accl[l][t]);
      if (lane == 0) red[wave * NRED + KK * (l + 1) + t] = v;
    }
  {
    const float v = wave_sum(gsum);
    if (lane == 0) red[wave * NRED + NRED - 1] = v;
  }
  __syncthreads();
  float* dst = partial + (static_cast<size_t>(chunk) * pl.C + c) * (NF * KK + 1);
  for (int o = tid; o < NF * KK + 1; o += blockDim.x) {
    float v = 0.f;
    if (o == NF * KK) {
      for (int wv = 0; wv < 8; ++wv) v += red[wv * NRED + NRED - 1];
    } else {
      const int f = o / KK, t = o - f * KK;
      if (f == 0) {
        for (int wv = 0; wv < 8; ++wv) v += red[wv * NRED + t];
      } else {
        const int l = (f - 1) >> 2, s = (f - 1) & 3;
        v = red[s * NRED + KK * (l + 1) + t] + red[(s + 4) * NRED + KK * (l + 1) + t];
      }
    }
    dst[o] = v;
  }
}

// Second stage: sum the per-chunk partials and apply the chain rule of the folding
//   dw = gamma * dWt,  dgamma = sum_t w * dWt (+ bias * sumG for the base scale),
//   dbias = gamma_b * sumG        (cf. fast_wtconv/cuda_haar/haar_cuda.py:168-197,657-676)
// One workgroup per channel, one thread per (filter, tap); the per-filter dot products go
// through LDS.  S = 4 (2-D) or 2 (1-D).  blockDim.x >= NF, dynamic LDS NF*KK floats.
__global__ void wgrad_finish_kernel(const float* __restrict__ partial, int nchunk, ParamTable p,
                                    int pdtype, GradTable gt, int C, int S, int L, int KK) {
  WT_SHARED_FLOATS(prod);
  const int NF = 1 + S * L;
  const int stride = NF * KK + 1;
  const int c = blockIdx.x;
  for (int o = threadIdx.x; o < NF * KK; o += blockDim.x) {
    float sum = 0.f;
    for (int ch = 0; ch < nchunk; ++ch) sum += partial[(static_cast<size_t>(ch) * C + c) * stride + o];
    const int f = o / KK, t = o - f * KK;
    float gam, wv;
    if (f == 0) {
      gam = load_param(p.base_scale, pdtype, c);
      wv = load_param(p.base_weight, pdtype, c * KK + t);
      gt.base_weight[c * KK + t] = gam * sum;
    } else {
      const int l = (f - 1) / S, chn = c * S + (f - 1) % S;
      gam = load_param(p.wt_scale[l], pdtype, chn);
      wv = load_param(p.wt_weight[l], pdtype, chn * KK + t);
      gt.wt_weight[l][chn * KK + t] = gam * sum;
    }
    prod[o] = wv * sum;
  }
  const int o = threadIdx.x;
  __syncthreads();
  if (o < NF) {
    float dot = 0.f;
    for (int t = 0; t < KK; ++t) dot += prod[o * KK + t];
    if (o == 0) {
      // sumG sits in the last slot of the channel's partial record
      float sg = 0.f;
      for (int ch = 0; ch < nchunk; ++ch) sg += partial[(static_cast<size_t>(ch) * C + c) * stride + NF * KK];
      if (p.base_bias != nullptr) {
        dot = fmaf(load_param(p.base_bias, pdtype, c), sg, dot);
        if (gt.base_bias != nullptr) gt.base_bias[c] = load_param(p.base_scale, pdtype, c) * sg;
      }
      gt.base_scale[c] = dot;
    } else {
      const int l = (o - 1) / S, chn = c * S + (o - 1) % S;
      gt.wt_scale[l][chn] = dot;
    }
  }
}

}  // namespace wt
