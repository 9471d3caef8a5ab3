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
#include "wgrad_finish.h"

namespace wt {

constexpr int kFetchPasses = 2;  // 2x4 pieces of the next plane a thread may hold in registers

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
  int vec_ok;                  // W % 4 == 0 and every tensor pointer aligned to 4 elements:
                               //   rows can be moved as 4-element vectors
  int prefetch;                // vec_ok and a plane is at most kFetchPasses pieces per thread:
                               //   the next plane is fetched into registers during compute
  int nplanes;                 // B * C
  int B;
  int sg_shift;                // log2 of the threads that share one plane (4..8)
  int plane_lds_floats;        // LDS of one plane slot; lds_floats = slots * this
  int groups_per_channel;      // sg < 64: a wave holds 64/sg planes of one channel; number of such groups per channel
  int fuse;                    // deepest analysis level produced from registers at commit (1..3)
  int block;                   // plane kernel: threads per workgroup (256, or 512 = two whole-workgroup planes)
  int pb;                      // weight-gradient kernel: planes of one channel stacked per iteration
  int slot_shift;              //   log2 of the threads that load/analyse one of them
};

// ------------------------------------------------------------------ parameter folding
// fw[c][f][t]: f = 0 base conv, f = 1 + S*l + s level l sub-band s; value gamma * w, taps
// reversed when flip != 0.  fb[c] = gamma_b * bias (0 without bias).  Also clears the `nzero` words at `zero_words`
// (the channel tickets of a parameter-gradient pass that follows on the stream).
__global__ void fold_params_kernel(ParamTable p, int pdtype, float* __restrict__ fw,
                                   float* __restrict__ fb, int C, int S, int L, int KK,
                                   int flip, int use_bias, unsigned* __restrict__ zero_words, int nzero) {
  const int NF = 1 + S * L;
  const int total = C * NF * KK;
  for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < nzero; i += gridDim.x * blockDim.x) zero_words[i] = 0u;
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

// Synchronisation between the phases of a plane: workgroup barrier, or only the ordering of
// one wave's LDS traffic when every plane belongs to the lanes of a single wave.
__device__ __forceinline__ void plane_sync(bool wave_local) {
  if (wave_local) WT_WAVE_LDS_SYNC();
  else WT_LDS_BARRIER();
}

// ------------------------------------------------------------------ plane load
// Copy one contiguous H x W plane from HBM into a haloed (or padded) LDS buffer whose
// element (r, col) sits at dst[(r + P) * str + col + P].
template <typename T>
__device__ __forceinline__ void load_plane(const T* __restrict__ src, float* __restrict__ dst,
                                           int H, int W, int str, int P, int tid, int nthreads,
                                           bool valid = true) {
  const int gsh = W <= 1 ? 0 : 32 - __clz(W - 1);
  const int rpp = nthreads >> gsh;
  if (rpp >= 1) {                      // lane groups of 2^gsh >= W lanes walk whole rows
    const int col = tid & ((1 << gsh) - 1);
    if (col >= W || (tid >> gsh) >= rpp) return;
    for (int r = tid >> gsh; r < H; r += rpp)
      dst[(r + P) * str + col + P] = valid ? to_f32<T>(src[r * W + col]) : 0.f;
  } else {
    const int n = H * W;
    for (int e = tid; e < n; e += nthreads) {
      const int r = e / W, col = e - r * W;
      dst[(r + P) * str + col + P] = valid ? to_f32<T>(src[e]) : 0.f;
    }
  }
}

// Lane grouping without divisions: a level whose rows hold `nitem` work items is walked by
// groups of GS = 2^gsh >= nitem consecutive lanes, one row per group and pass.  Lanes of a
// group touch one LDS row at consecutive addresses.
__device__ __forceinline__ int group_shift(int nitem) {
  return nitem <= 1 ? 0 : 32 - __clz(nitem - 1);
}

// Four consecutive elements from HBM (address aligned to 4 elements).
template <typename T>
__device__ __forceinline__ void load4(const T* __restrict__ p, float (&v)[4]) {
  if constexpr (sizeof(T) == 4) {
    const float4 q = *reinterpret_cast<const float4*>(p);
    v[0] = q.x; v[1] = q.y; v[2] = q.z; v[3] = q.w;
  } else {
    const uint2 q = *reinterpret_cast<const uint2*>(p);
    unpack2<T>(q.x, v[0], v[1]);
    unpack2<T>(q.y, v[2], v[3]);
  }
}

// Fused plane load + first analysis level for planes whose width is a multiple of 4:
// a work item owns 2 input rows x 4 input columns (2 level-1 positions); it copies them
// into the level-0 buffer and writes the four level-1 sub-bands, so the plane is read from
// HBM with 16-byte (fp32) / 8-byte (bf16) loads and never re-read from LDS for level 1.
// Odd H: the missing bottom row is the zero padding of wtconv2d.py:49-51.
template <typename T>
__device__ __forceinline__ void load_analysis1(const T* __restrict__ src, int H, int W,
                                               float* __restrict__ d0, int str0, int P0,
                                               float* __restrict__ d1, int str1, int pl1, int P1,
                                               int tid, int nthreads, bool valid = true) {
  const int h1 = (H + 1) >> 1;
  const int nitem = W >> 2;                     // 4-column pieces per row
  const int gsh = group_shift(nitem);
  const int s = tid & ((1 << gsh) - 1);
  if (s >= nitem) return;
  const int c0 = 4 * s;
  for (int i = tid >> gsh; i < h1; i += nthreads >> gsh) {
    float a[4] = {0.f, 0.f, 0.f, 0.f}, b[4] = {0.f, 0.f, 0.f, 0.f};
    const bool has_b = 2 * i + 1 < H;
    if (valid) {
      load4<T>(src + imul(2 * i, W) + c0, a);
      if (has_b) load4<T>(src + imul(2 * i + 1, W) + c0, b);
    }
    float* x0 = d0 + imul(2 * i + P0, str0) + c0 + P0;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      x0[k] = a[k];
      if (has_b) x0[str0 + k] = b[k];
    }
    float* o = d1 + imul(i + P1, str1) + 2 * s + P1;
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const float sac = a[2 * t] + b[2 * t], sbd = a[2 * t + 1] + b[2 * t + 1];
      const float dac = a[2 * t] - b[2 * t], dbd = a[2 * t + 1] - b[2 * t + 1];
      o[t] = 0.5f * (sac + sbd);
      o[pl1 + t] = 0.5f * (dac + dbd);
      o[2 * pl1 + t] = 0.5f * (sac - sbd);
      o[3 * pl1 + t] = 0.5f * (dac - dbd);
    }
  }
}

// The same work split in two, so that the HBM reads of the next plane are in flight while
// the current one is computed: plane_fetch issues the loads into registers (NP passes of
// one 2x4 piece per thread), plane_commit writes level 0 and level 1 into LDS.
template <typename T, int NP>
__device__ __forceinline__ void plane_fetch(const T* __restrict__ src, int H, int W, int tid, int nthreads,
                                            float (&a)[NP][4], float (&b)[NP][4]) {
  const int h1 = (H + 1) >> 1;
  const int nitem = W >> 2;
  const int gsh = group_shift(nitem);
  const int s = tid & ((1 << gsh) - 1);
  if (s >= nitem) return;
  const int c0 = 4 * s;
#pragma unroll
  for (int p = 0; p < NP; ++p) {
    const int i = (tid >> gsh) + p * (nthreads >> gsh);
    if (i < h1) {
      // both loads unconditional (no merge with constants, hence no wait right behind the
      // load); a missing bottom row re-reads the top one and is zeroed in plane_commit
      const int rb = 2 * i + 1 < H ? 2 * i + 1 : 2 * i;
      load4<T>(src + imul(2 * i, W) + c0, a[p]);
      load4<T>(src + imul(rb, W) + c0, b[p]);
    }
  }
}

template <int NP>
__device__ __forceinline__ void plane_commit(const float (&a)[NP][4], const float (&b)[NP][4], int H, int W,
                                             float* __restrict__ d0, int str0, int P0,
                                             float* __restrict__ d1, int str1, int pl1, int P1,
                                             int tid, int nthreads, bool valid = true) {
  const int h1 = (H + 1) >> 1;
  const int nitem = W >> 2;
  const int gsh = group_shift(nitem);
  const int s = tid & ((1 << gsh) - 1);
  if (s >= nitem) return;
  const int c0 = 4 * s;
#pragma unroll
  for (int p = 0; p < NP; ++p) {
    const int i = (tid >> gsh) + p * (nthreads >> gsh);
    if (i < h1) {
      const bool has_b = 2 * i + 1 < H;
      float aa[4], bb[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) {      // a slot without a plane commits zeros
        aa[k] = valid ? a[p][k] : 0.f;
        bb[k] = (valid && has_b) ? b[p][k] : 0.f;
      }
      float* x0 = d0 + imul(2 * i + P0, str0) + c0 + P0;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        x0[k] = aa[k];
        if (has_b) x0[str0 + k] = bb[k];
      }
      float* o = d1 + imul(i + P1, str1) + 2 * s + P1;
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const float sac = aa[2 * t] + bb[2 * t], sbd = aa[2 * t + 1] + bb[2 * t + 1];
        const float dac = aa[2 * t] - bb[2 * t], dbd = aa[2 * t + 1] - bb[2 * t + 1];
        o[t] = 0.5f * (sac + sbd);
        o[pl1 + t] = 0.5f * (dac + dbd);
        o[2 * pl1 + t] = 0.5f * (sac - sbd);
        o[3 * pl1 + t] = 0.5f * (dac - dbd);
      }
    }
  }
}

// plane_commit that also produces levels 2 (and 3) straight from the registers: with the
// lane layout (row-pair i, piece s) = (lane >> gsh, lane & (2^gsh - 1)) the 2x2 block of
// level-1 LL values behind a level-2 coefficient sits in lanes i and i^1, and the level-2
// block behind a level-3 coefficient in lanes (i, s), (i, s^1), (i^2, s), (i^2, s^1) of the
// same wavefront, so wavefront shuffles replace two LDS round trips and two barriers per
// plane.  Needs 2^gsh <= 16 lanes per row (so that 4 row-pairs share a wave) and every lane
// of the wave in the call; lanes without a piece contribute zeros, which is also the
// zero padding of odd sizes.  `fuse` = deepest level produced (2 or 3).
template <int NP>
__device__ __forceinline__ void plane_commit_fused(const float (&a)[NP][4], const float (&b)[NP][4], int H, int W,
                                                   float* __restrict__ d0, int str0, int P0,
                                                   float* __restrict__ d1, int str1, int pl1,
                                                   float* __restrict__ d2, int str2, int pl2,
                                                   float* __restrict__ d3, int str3, int pl3, int P1,
                                                   int fuse, int tid, int nthreads) {
  const int h1 = (H + 1) >> 1;
  const int nitem = W >> 2;
  const int gsh = group_shift(nitem);
  const int s = tid & ((1 << gsh) - 1);
  const int c0 = 4 * s;
  const int lane4 = (tid & (kWave - 1)) << 2;
#pragma unroll
  for (int p = 0; p < NP; ++p) {
    const int i = (tid >> gsh) + p * (nthreads >> gsh);
    const bool valid = s < nitem && i < h1;
    const bool has_b = 2 * i + 1 < H;
    float aa[4], bb[4], ll1[2];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      aa[k] = valid ? a[p][k] : 0.f;
      bb[k] = (valid && has_b) ? b[p][k] : 0.f;
    }
    if (valid) {
      float* x0 = d0 + imul(2 * i + P0, str0) + c0 + P0;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        x0[k] = aa[k];
        if (has_b) x0[str0 + k] = bb[k];
      }
    }
    float* o1 = d1 + imul(i + P1, str1) + 2 * s + P1;
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const float sac = aa[2 * t] + bb[2 * t], sbd = aa[2 * t + 1] + bb[2 * t + 1];
      const float dac = aa[2 * t] - bb[2 * t], dbd = aa[2 * t + 1] - bb[2 * t + 1];
      ll1[t] = 0.5f * (sac + sbd);
      if (valid) {
        o1[t] = ll1[t];
        o1[pl1 + t] = 0.5f * (dac + dbd);
        o1[2 * pl1 + t] = 0.5f * (sac - sbd);
        o1[3 * pl1 + t] = 0.5f * (dac - dbd);
      }
    }
    // level 2: rows i (even) and i+1 of level 1
    const float bot0 = wave_xor(ll1[0], lane4, 1 << gsh);
    const float bot1 = wave_xor(ll1[1], lane4, 1 << gsh);
    const bool own2 = valid && (i & 1) == 0;
    float ll2;
    {
      const float sac = ll1[0] + bot0, sbd = ll1[1] + bot1, dac = ll1[0] - bot0, dbd = ll1[1] - bot1;
      ll2 = own2 ? 0.5f * (sac + sbd) : 0.f;
      if (own2) {
        float* o2 = d2 + imul((i >> 1) + P1, str2) + s + P1;
        o2[0] = ll2;
        o2[pl2] = 0.5f * (dac + dbd);
        o2[2 * pl2] = 0.5f * (sac - sbd);
        o2[3 * pl2] = 0.5f * (dac - dbd);
      }
    }
    if (fuse >= 3) {   // level 3: level-2 positions (i/2, s), (i/2, s+1), (i/2+1, s), (i/2+1, s+1)
      const float right = wave_xor(ll2, lane4, 1);
      const float down = wave_xor(ll2, lane4, 2 << gsh);
      const float diag = wave_xor(right, lane4, 2 << gsh);
      if (valid && (i & 3) == 0 && (s & 1) == 0) {
        const float sac = ll2 + down, sbd = right + diag, dac = ll2 - down, dbd = right - diag;
        float* o3 = d3 + imul((i >> 2) + P1, str3) + (s >> 1) + P1;
        o3[0] = 0.5f * (sac + sbd);
        o3[pl3] = 0.5f * (dac + dbd);
        o3[2 * pl3] = 0.5f * (sac - sbd);
        o3[3 * pl3] = 0.5f * (dac - dbd);
      }
    }
  }
}

// One analysis level: src is the (haloed/padded, zero outside) LL plane of level l-1,
// dst the four sub-band planes of level l.  Reading one past the source grid returns the
// zero padding the reference applies to odd sizes (wtconv2d.py:49-51).
__device__ __forceinline__ void analysis_level(const float* __restrict__ src, int sstr, int sP,
                                               float* __restrict__ dst, int dstr, int dpl, int dP,
                                               int hl, int wl, int tid, int nthreads) {
  const int gsh = group_shift(wl);
  const int rpp = nthreads >> gsh;
  if (rpp == 0) {   // a row is wider than the lane group: plain strided walk
    for (int it = tid; it < hl * wl; it += nthreads) {
      const int i = it / wl, j = it - i * wl;
      const float* s0 = src + imul(2 * i + sP, sstr) + 2 * j + sP;
      const float a = s0[0], b = s0[1], c = s0[sstr], d = s0[sstr + 1];
      const float sac = a + c, sbd = b + d, dac = a - c, dbd = b - d;
      float* o = dst + imul(i + dP, dstr) + j + dP;
      o[0] = 0.5f * (sac + sbd);
      o[dpl] = 0.5f * (dac + dbd);
      o[2 * dpl] = 0.5f * (sac - sbd);
      o[3 * dpl] = 0.5f * (dac - dbd);
    }
    return;
  }
  const int j = tid & ((1 << gsh) - 1);
  if (j >= wl) return;
  for (int i = tid >> gsh; i < hl; i += rpp) {
    const float* s0 = src + imul(2 * i + sP, sstr) + 2 * j + sP;
    const float a = s0[0], b = s0[1], c = s0[sstr], d = s0[sstr + 1];
    const float sac = a + c, sbd = b + d, dac = a - c, dbd = b - d;
    float* o = dst + imul(i + dP, dstr) + j + dP;
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
// K x K correlation of TJ horizontally adjacent outputs; `a` points at the top-left input
// of the first output's window (VW*4-byte aligned).  One call is one "chunk": its K row
// reads are what the compiler may keep in flight at once.
template <int K, int TJ, int VW>
__device__ __forceinline__ void conv_strip(const float* __restrict__ a, int astr,
                                           wt_uniform_ptr wf, float (&y)[TJ]) {
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

// Conv of sub-band S of TJ coefficient quads: one fenced chunk.
template <int K, int TJ, int VW, int S>
__device__ __forceinline__ void subband_conv(const float* __restrict__ a, int astr, int apl, wt_uniform_ptr wf,
                                             float (&y)[TJ]) {
#pragma unroll
  for (int t = 0; t < TJ; ++t) y[t] = 0.f;
  wt_uniform_ptr w = wf + S * K * K;
  WT_LAUNDER_UNIFORM_PTR(w);
  conv_strip<K, TJ, VW>(a + S * apl, astr, w, y);
}

// The four sub-band convolutions of TJ coefficient quads and the inverse Haar butterflies:
// o0 / o1 receive the 2 x 2TJ reconstructed samples scaled by 2 (the caller applies the 1/2).
// Two butterfly stages (LL +- LH as soon as both exist, then +- (HL +- HH)): 8 additions per
// quad.  One fenced chunk per sub-band bounds the LDS rows in flight.
template <int K, int TJ, int VW>
__device__ __forceinline__ void subband_chunks(const float* __restrict__ a, int astr, int apl,
                                               wt_uniform_ptr wf, const float* __restrict__ zin,
                                               float (&o0)[2 * TJ], float (&o1)[2 * TJ]) {
  float p[TJ], m[TJ];
  {
    float ll[TJ];
    subband_conv<K, TJ, VW, 0>(a, astr, apl, wf, ll);
    if (zin != nullptr) {
#pragma unroll
      for (int t = 0; t < TJ; ++t) ll[t] += zin[t];
    }
    pin_values(ll);
    WT_CHUNK_FENCE();
    float lh[TJ];
    subband_conv<K, TJ, VW, 1>(a, astr, apl, wf, lh);
#pragma unroll
    for (int t = 0; t < TJ; ++t) { p[t] = ll[t] + lh[t]; m[t] = ll[t] - lh[t]; }
    pin_values(p);
    pin_values(m);
    WT_CHUNK_FENCE();
  }
  float hl[TJ];
  subband_conv<K, TJ, VW, 2>(a, astr, apl, wf, hl);
  pin_values(hl);
  WT_CHUNK_FENCE();
  float hh[TJ];
  subband_conv<K, TJ, VW, 3>(a, astr, apl, wf, hh);
#pragma unroll
  for (int t = 0; t < TJ; ++t) {
    const float q = hl[t] + hh[t], n = hl[t] - hh[t];
    o0[2 * t] = p[t] + q;
    o0[2 * t + 1] = p[t] - q;
    o1[2 * t] = m[t] + n;
    o1[2 * t + 1] = m[t] - n;
  }
  pin_values(o0);
  pin_values(o1);
  WT_CHUNK_FENCE();
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
                                            wt_uniform_ptr wl_f, int ltid, int nth) {
  constexpr int R = K / 2;
  constexpr int VW = (R >= 1) ? TJ : 1;   // window starts at column j0 when the halo equals R
  const int hl = pl.h[l], wl = pl.w[l];
  const int nstrip = (wl + TJ - 1) / TJ;
  const int gsh = group_shift(nstrip);
  const int strip = ltid & ((1 << gsh) - 1);
  if (strip >= nstrip) return;
  const int j0 = strip * TJ;
  const int astr = pl.astr[l], apl = pl.apl[l], P = pl.P;
  const float* A = lds + pl.aoff[l];
  const bool has_carry = l < pl.L;
  const float* Zin = lds + pl.zoff[l + 1];
  const int zin_str = pl.zstr[l + 1];
  float* Zout = lds + pl.zoff[l];
  const int zout_str = pl.zstr[l];
  const int ho = pl.h[l - 1], wo = pl.w[l - 1];
  const int rpp = (nth >> gsh) > 0 ? (nth >> gsh) : 1;
  if ((ltid >> gsh) >= rpp) return;            // more strips than lanes: not used (nth >= 16 >= strips)
  for (int i = ltid >> gsh; i < hl; i += rpp) {
    float o0[2 * TJ], o1[2 * TJ];
    subband_chunks<K, TJ, VW>(A + imul(i - R + P, astr) + (j0 - R + P), astr, apl, wl_f,
                                 has_carry ? Zin + imul(i, zin_str) + j0 : nullptr, o0, o1);
    const int r0 = 2 * i;
#pragma unroll
    for (int t = 0; t < 2 * TJ; ++t) {
      const int c0 = 2 * j0 + t;
      if (c0 < wo) {
        Zout[imul(r0, zout_str) + c0] = 0.5f * o0[t];
        if (r0 + 1 < ho) Zout[imul(r0 + 1, zout_str) + c0] = 0.5f * o1[t];
      }
    }
  }
}

// Store up to N consecutive outputs (`nvalid` of them lie inside the row): 4-element vectors
// when the whole strip is inside, the destination is aligned to 4 elements and vec4 is set.
template <typename T, int N>
__device__ __forceinline__ void store_row(T* __restrict__ dst, const float (&v)[N], int nvalid, bool vec4) {
  if constexpr (N % 4 == 0) {
    if (vec4 && nvalid == N) {           // the common case: whole strip inside the row, 16-byte stores
#pragma unroll
      for (int k = 0; k < N / 4; ++k) {
        if constexpr (sizeof(T) == 4) {
          float4 q;
          q.x = v[4 * k]; q.y = v[4 * k + 1]; q.z = v[4 * k + 2]; q.w = v[4 * k + 3];
          *reinterpret_cast<float4*>(dst + 4 * k) = q;
        } else {
          uint2 q;
          q.x = pack2<T>(v[4 * k], v[4 * k + 1]);
          q.y = pack2<T>(v[4 * k + 2], v[4 * k + 3]);
          *reinterpret_cast<uint2*>(dst + 4 * k) = q;
        }
      }
      return;
    }
  }
#pragma unroll
  for (int e = 0; e < N; ++e)
    if (e < nvalid) dst[e] = from_f32<T>(v[e]);
}

// Level 1: conv of the four sub-bands, add Z_2, inverse Haar, add the scaled base conv
// (and bias) of the same 2 x 2TJ pixels, store to HBM.
template <typename T, int K, int TJ>
__device__ __forceinline__ void synth_final(float* __restrict__ lds, const Plan2D& pl,
                                            wt_uniform_ptr wb_f, wt_uniform_ptr w1_f, float bias,
                                            T* __restrict__ out_plane, int ltid, int nth) {
  constexpr int R = K / 2;
  constexpr int NO = 2 * TJ;
  constexpr int VW = (R >= 1) ? TJ : 1;
  constexpr int VWX = (R >= 1) ? (NO >= 4 ? 4 : NO) : 1;
  const int hl = pl.h[1], wl = pl.w[1];
  const int nstrip = (wl + TJ - 1) / TJ;
  const int gsh = group_shift(nstrip);
  const int strip = ltid & ((1 << gsh) - 1);
  if (strip >= nstrip) return;
  const int j0 = strip * TJ;
  const int astr = pl.astr[1], apl = pl.apl[1], P = pl.P;
  const float* A = lds + pl.aoff[1];
  const float* X = lds + pl.aoff[0];
  const int xstr = pl.astr[0];
  const bool has_carry = pl.L > 1;
  const float* Zin = lds + pl.zoff[2];
  const int zin_str = pl.zstr[2];
  const int H = pl.H, W = pl.W;
  const int rpp = (nth >> gsh) > 0 ? (nth >> gsh) : 1;
  if ((ltid >> gsh) >= rpp) return;
  for (int i = ltid >> gsh; i < hl; i += rpp) {
    float o0[NO], o1[NO];
    subband_chunks<K, TJ, VW>(A + imul(i - R + P, astr) + (j0 - R + P), astr, apl, w1_f,
                                 has_carry ? Zin + imul(i, zin_str) + j0 : nullptr, o0, o1);
#pragma unroll
    for (int t = 0; t < NO; ++t) { o0[t] = fmaf(0.5f, o0[t], bias); o1[t] = fmaf(0.5f, o1[t], bias); }
    // base conv of output rows 2i, 2i+1, columns 2j0 .. 2j0+NO-1, accumulated on top; input
    // row r feeds output row 0 through kernel row r and output row 1 through kernel row r-1
    const float* xw = X + imul(2 * i - R + P, xstr) + (2 * j0 - R + P);
    constexpr int NRX = pad_to(NO + K - 1, VWX);
    wt_uniform_ptr wb = wb_f;
    WT_LAUNDER_UNIFORM_PTR(wb);
#pragma unroll
    for (int r = 0; r < K + 1; ++r) {
      float row[NRX];
      lds_row<NRX, VWX>(xw + r * xstr, row);
      if (r < K) {
#pragma unroll
        for (int kw = 0; kw < K; ++kw) {
          const float wv = wb[r * K + kw];
#pragma unroll
          for (int t = 0; t < NO; ++t) o0[t] = fmaf(wv, row[t + kw], o0[t]);
        }
      }
      if (r >= 1) {
#pragma unroll
        for (int kw = 0; kw < K; ++kw) {
          const float wv = wb[(r - 1) * K + kw];
#pragma unroll
          for (int t = 0; t < NO; ++t) o1[t] = fmaf(wv, row[t + kw], o1[t]);
        }
      }
      if (r == K / 2) {
        pin_values(o0);
        pin_values(o1);
        WT_CHUNK_FENCE();
      }
    }
    const int r0 = 2 * i, c0 = 2 * j0;
    int nvalid = W - c0;
    if (nvalid > NO) nvalid = NO;
    pin_values(o0);      // all outputs computed before the stores: keeps the compiler from sinking
    pin_values(o1);      // the last FMAs behind the store branches and splitting the 16-byte stores
    if (nvalid > 0) {
      store_row<T, NO>(out_plane + imul(r0, W) + c0, o0, nvalid, pl.vec_ok != 0);
      if (r0 + 1 < H) store_row<T, NO>(out_plane + imul(r0 + 1, W) + c0, o1, nvalid, pl.vec_ok != 0);
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
// Persistent: grid.x = min(work units, resident workgroups), block = 256 or 512 threads.
// 2^sg_shift threads share a plane, so a workgroup holds blockDim >> sg_shift planes, each in
// its own LDS slot (small planes: up to 16 per workgroup; planes that take 256 threads run
// two to a workgroup, which halves the barrier-bound cost of their small coarse levels).  When a plane takes less than a wave,
// the planes of one wave are the same channel of consecutive batch items, so the folded
// weights stay wave-uniform (SGPRs).  The zero halos written once stay valid for every plane
// (only interiors are rewritten).
// MODE selects the loader at compile time (0: register prefetch of the next plane, 3: the same
// with levels 2-3 produced at the commit, 1: fused vector load without prefetch, 2: element-wise
// load), so that the hot variant does not carry
// the registers of the others.
// Geo: the plan's geometry as a compile-time constant for the common shapes (LDS offsets and strides fold into
// instruction immediates, loops over levels unroll), or the run-time plan of the argument for any other shape;
// batch, channels and what follows from them always come from the argument.
template <typename T, int K, int TJ1, int TJC, int MODE, typename Geo>
__global__ __launch_bounds__(512, 4) void wt2d_plane_kernel(const T* __restrict__ x, T* __restrict__ out,
                                                         const float* __restrict__ fw,
                                                         const float* __restrict__ fb, const Plan2D plarg) {
  WT_SHARED_FLOATS(lds_all);
  static constexpr Plan2D kGeo = Geo::plan();
  const Plan2D& pl = Geo::kStatic ? kGeo : plarg;
  const int nB = plarg.B, nC = plarg.C, nplanes = plarg.nplanes, gpc = plarg.groups_per_channel;
  constexpr int KK = K * K;
  const int NF = 1 + 4 * pl.L;
  const size_t plane_elems = static_cast<size_t>(pl.H) * pl.W;
  const int tid = threadIdx.x;
  const int sg = 1 << pl.sg_shift;
  int ltid = tid & (sg - 1);
  const int slot = tid >> pl.sg_shift;
  const int slots = blockDim.x >> pl.sg_shift;
  float* lds = lds_all + slot * pl.plane_lds_floats;
  const int wave = tid >> 6;
  const int ppw = sg < kWave ? kWave >> pl.sg_shift : 1;      // planes per wave
  const int nunits = sg < kWave ? (nC * gpc + 3) / 4 : (nplanes + slots - 1) / slots;

  // Plane of this thread in a work unit (-1: none) and its (wave-uniform) channel.  The
  // divisions happen once: `locate` positions the state on the workgroup's first unit, and
  // `advance` moves it by gridDim.x units with additions and one compare (a 32-bit integer
  // division costs ~35 vector instructions, several of them quarter rate).
  struct Loc { int plane, c, key, rem; };       // key: un-clamped plane (sg >= 64); rem: gidx % groups (sg < 64)
  const int G = gridDim.x;
  int step_c = 0, step_q = 0, step_r = 0;
  if (sg < kWave) {
    step_q = (4 * G) / gpc;
    step_r = 4 * G - step_q * gpc;
  } else {
    step_c = static_cast<int>((static_cast<long long>(G) * slots) % nC);
  }
  auto resolve = [&](Loc& s) {
    if (sg < kWave) {
      const int b = imul(s.rem, ppw) + ((tid & (kWave - 1)) >> pl.sg_shift);
      s.plane = (s.c < nC && b < nB) ? imul(b, nC) + s.c : -1;
    } else {
      s.plane = s.key < nplanes ? s.key : -1;
    }
  };
  auto locate = [&](int u, Loc& s) {
    if (sg < kWave) {
      const int gidx = u * 4 + wave;
      s.c = gidx / gpc;
      s.rem = gidx - s.c * gpc;
      s.key = 0;
    } else {
      s.key = u * slots + slot;
      s.c = s.key % nC;
      s.rem = 0;
    }
    resolve(s);
  };
  auto advance = [&](Loc& s) {
    if (sg < kWave) {
      s.c += step_q;
      s.rem += step_r;
      if (s.rem >= gpc) { s.rem -= gpc; s.c += 1; }
    } else {
      s.key += G * slots;           // may pass nplanes: resolve() maps that to "no plane"
      s.c += step_c;
      if (s.c >= nC) s.c -= nC;
    }
    resolve(s);
  };
  // the channel used for the weights (clamped: a thread without a plane still runs uniform code)
  auto channel_of = [&](const Loc& s) { return s.c < nC ? s.c : nC - 1; };

  constexpr bool kPrefetch = MODE == 0 || MODE == 3;
  float fa[kFetchPasses][4], fbuf[kFetchPasses][4];
  Loc nxt;
  locate(blockIdx.x, nxt);
  if (kPrefetch && nxt.plane >= 0)
    plane_fetch<T, kFetchPasses>(x + nxt.plane * plane_elems, pl.H, pl.W, ltid, sg, fa, fbuf);
  zero_lds(lds_all, pl.lds_floats);      // while the first plane is on its way from HBM
  WT_LDS_BARRIER();
  // Every path into the loop body has now waited for its prefetch (here, and before the stores
  // of the final phase below), so the commit at the top of the body needs no vmcnt wait of its
  // own -- which would also wait for the stores of the previous plane.
  WT_WAIT_VMEM();
  // A plane owned by the lanes of one wave needs no workgroup barrier between its phases: the
  // waves of the workgroup drift apart and fill each other's latency-bound phases.
  const bool wave_local = pl.sg_shift <= 6;
  for (int uv = blockIdx.x; uv < nunits; uv += gridDim.x) {
    const int u = WT_UNIFORM(uv);
    const int plane = nxt.plane;
    const int c = WT_UNIFORM(channel_of(nxt));
    const bool live = plane >= 0;
    advance(nxt);
    wt_uniform_ptr fwc = (wt_uniform_ptr)(fw + static_cast<size_t>(c) * NF * KK);
    const size_t plane_off = static_cast<size_t>(live ? plane : 0) * plane_elems;
    int l0 = 2;
    WT_WAVE_PRIORITY(3);
    if constexpr (MODE == 0) {
      if (live)
        plane_commit<kFetchPasses>(fa, fbuf, pl.H, pl.W, lds + pl.aoff[0], pl.astr[0], pl.P,
                                   lds + pl.aoff[1], pl.astr[1], pl.apl[1], pl.P, ltid, sg);
    } else if constexpr (MODE == 3) {   // one plane per workgroup: `live` is uniform
      if (live) {
        plane_commit_fused<kFetchPasses>(fa, fbuf, pl.H, pl.W, lds + pl.aoff[0], pl.astr[0], pl.P, lds + pl.aoff[1],
                                         pl.astr[1], pl.apl[1], lds + pl.aoff[2], pl.astr[2], pl.apl[2],
                                         lds + pl.aoff[pl.fuse], pl.astr[pl.fuse], pl.apl[pl.fuse], pl.P, pl.fuse,
                                         ltid, sg);
        l0 = pl.fuse + 1;
      }
    } else if constexpr (MODE == 1) {
      if (live)
        load_analysis1<T>(x + plane_off, pl.H, pl.W, lds + pl.aoff[0], pl.astr[0], pl.P,
                          lds + pl.aoff[1], pl.astr[1], pl.apl[1], pl.P, ltid, sg);
    } else {
      if (live) load_plane<T>(x + plane_off, lds + pl.aoff[0], pl.H, pl.W, pl.astr[0], pl.P, ltid, sg);
      l0 = 1;
    }
    plane_sync(wave_local);
    if (kPrefetch && u + static_cast<int>(gridDim.x) < nunits && nxt.plane >= 0)
      plane_fetch<T, kFetchPasses>(x + nxt.plane * plane_elems, pl.H, pl.W, ltid, sg, fa, fbuf);
    for (int lv = l0; lv <= pl.L; ++lv) {
      const int l = WT_UNIFORM(lv);
      if (live)
        analysis_level(lds + pl.aoff[l - 1], pl.astr[l - 1], pl.P, lds + pl.aoff[l], pl.astr[l], pl.apl[l], pl.P,
                       pl.h[l], pl.w[l], ltid, sg);
      plane_sync(wave_local);
    }
    for (int lv = pl.L; lv >= 2; --lv) {
      const int l = WT_UNIFORM(lv);
      if (live) synth_inner<K, TJC>(lds, pl, l, fwc + (1 + 4 * (l - 1)) * KK, ltid, sg);
      plane_sync(wave_local);
    }
    WT_WAIT_VMEM();     // next plane's loads have landed; the stores below are not waited for
    WT_WAVE_PRIORITY(0);
    if (live) synth_final<T, K, TJ1>(lds, pl, fwc, fwc + KK, fb[c], out + plane_off, ltid, sg);
    plane_sync(wave_local);   // the next plane overwrites the buffers read above
  }
}

// ------------------------------------------------------------------ parameter gradients
// grid = (C, nchunk), block = 512 threads = 8 waves.  Each workgroup walks `bchunk`
// planes of one channel and keeps K*K correlation sums per filter in registers:
//   dWt_l[c,s,kh,kw] = sum_{b,i,j} dY_l[s][i,j] * A_l[s][i+kh-R, j+kw-R]
//   dWt_b[c,kh,kw]   = sum_{b,i,j} G[i,j] * x[i+kh-R, j+kw-R],   sumG[c] = sum G
// The filters are split over the waves so that no thread carries more than three sets:
//   waves 0-3 ("A", sub-band/quarter q = wave):   base conv rows of quarter q, level 3, level 5
//   waves 4-7 ("B", sub-band q = wave - 4):       level 1, level 2, level 4
// One cross-lane reduction at the end, partial sums to HBM, finished by
// wgrad_finish_kernel (two-stage and deterministic; the reference accumulates with float
// atomics, fused_haar_conv.cu:331-341).
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
    if (TJ > 1 && kh == K / 2 && K > 3) {   // two chunks per strip: at most (K+1)/2 rows in flight
      pin_values(acc);
      pin_values(dy);
      WT_CHUNK_FENCE();
    }
  }
  pin_values(acc);
  WT_CHUNK_FENCE();
}

// Two vertically adjacent strips at once: the K+1 input rows they span are read once, row r
// feeding kernel row r of the upper strip and kernel row r-1 of the lower one (a third
// fewer LDS reads per FMA than two separate strips).
template <int K, int TJ, int VW>
__device__ __forceinline__ void corr_strip2(const float* __restrict__ a, int astr,
                                            const float* __restrict__ gy0, const float* __restrict__ gy1,
                                            float (&acc)[K * K]) {
  constexpr int NR = pad_to(TJ + K - 1, VW);
  float dy0[TJ], dy1[TJ];
  lds_row<TJ, (TJ % 4 == 0) ? 4 : 1>(gy0, dy0);
  lds_row<TJ, (TJ % 4 == 0) ? 4 : 1>(gy1, dy1);
#pragma unroll
  for (int r = 0; r < K + 1; ++r) {
    float row[NR];
    lds_row<NR, VW>(a + r * astr, row);
    if (r < K) {
#pragma unroll
      for (int kw = 0; kw < K; ++kw) {
#pragma unroll
        for (int t = 0; t < TJ; ++t) acc[r * K + kw] = fmaf(dy0[t], row[t + kw], acc[r * K + kw]);
      }
    }
    if (r >= 1) {
#pragma unroll
      for (int kw = 0; kw < K; ++kw) {
#pragma unroll
        for (int t = 0; t < TJ; ++t) acc[(r - 1) * K + kw] = fmaf(dy1[t], row[t + kw], acc[(r - 1) * K + kw]);
      }
    }
    if (r == K / 2) {
      pin_values(acc);
      pin_values(dy0);
      pin_values(dy1);
      WT_CHUNK_FENCE();
    }
  }
  pin_values(acc);
  WT_CHUNK_FENCE();
}

// Correlation sums of one sub-band plane of one level, walked by a single wave.
// pass_row0/pass_step select the passes this wave owns (all: 0 / 1).  PAIR: work items are
// pairs of rows (the row below the last one must exist and hold zeros in G: it is the gap
// row under every stacked plane).
template <int K, int TJ, int VW, bool PAIR>
__device__ __forceinline__ void corr_level(const float* __restrict__ A, int astr, const float* __restrict__ G,
                                           int gstr, int h, int w, int lane, int pass_row0, int pass_step,
                                           float (&acc)[K * K]) {
  const int nstrip = (w + TJ - 1) / TJ;
  const int gsh = group_shift(nstrip);
  const int strip = lane & ((1 << gsh) - 1);
  if (strip >= nstrip) return;
  const int j0 = strip * TJ;
  const int rpp = kWave >> gsh;          // row items per pass of one wave (>= 1: nstrip <= 64)
  if constexpr (PAIR) {
    const int npair = (h + 1) >> 1;
    for (int ip = pass_row0 * rpp + (lane >> gsh); ip < npair; ip += pass_step * rpp) {
      const int i = 2 * ip;
      const float* gy = G + imul(i, gstr) + j0;
      corr_strip2<K, TJ, VW>(A + imul(i, astr) + j0, astr, gy, gy + gstr, acc);
    }
  } else {
    for (int i = pass_row0 * rpp + (lane >> gsh); i < h; i += pass_step * rpp) {
      const float* gy = G + imul(i, gstr) + j0;
      corr_strip<K, TJ, VW>(A + imul(i, astr) + j0, astr, gy, acc);   // A already points R rows/cols up-left
    }
  }
}

constexpr int wgrad_sets(int L) { return L >= 4 ? 3 : (L >= 2 ? 2 : 1); }
constexpr int kStripMinWidth = 12;   // coarse levels of the weight-gradient kernel: strips from this width on

template <typename T, int K, int L, int TJ, typename Geo>
__global__ __launch_bounds__(512, 4) void wt2d_wgrad_kernel(const T* __restrict__ x, const T* __restrict__ g,
                                                         float* __restrict__ partial, const Plan2D plarg,
                                                         int B, int bchunk, const FinishArgs fin) {
  WT_SHARED_FLOATS(lds);
  static constexpr Plan2D kGeo = Geo::plan();      // compile-time geometry for the common shapes (see wt2d_plane_kernel)
  const Plan2D& pl = Geo::kStatic ? kGeo : plarg;
  const int nC = plarg.C;
  constexpr int KK = K * K;
  constexpr int R = K / 2;
  constexpr int NF = 1 + 4 * L;
  constexpr int VW = (R >= 1 && TJ % 4 == 0) ? 4 : 1;
  constexpr int NSET = wgrad_sets(L);
  const int c = blockIdx.x;
  const int chunk = blockIdx.y;
  const int tid = threadIdx.x;
  const int wave = WT_UNIFORM(tid >> 6);
  int lane = tid & (kWave - 1);
  const int q = wave & 3;
  const bool role_a = wave < 4;
  const int P = pl.P;
  // `pb` planes (same channel, consecutive batch items) are stacked vertically per
  // iteration, separated by the P zero rows that already serve as halo: a correlation over
  // the stack is the sum of the per-plane correlations.  Slot k of the stack is loaded and
  // analysed by the threads with tid >> slot_shift == k.
  const int pb = pl.pb;
  int slot = tid >> pl.slot_shift;
  const int nps = 1 << pl.slot_shift;
  int ltid = tid & (nps - 1);
  const bool has_slot = slot < pb;
  const size_t plane_elems = static_cast<size_t>(pl.H) * pl.W;

  float acc[NSET][KK];
  float gsum = 0.f;
#pragma unroll
  for (int s = 0; s < NSET; ++s)
#pragma unroll
    for (int t = 0; t < KK; ++t) acc[s][t] = 0.f;


  // slot-local bases: level l of slot k starts k*(h_l+P) rows below the top of the stack
  auto a_slot = [&](int l) { return lds + pl.aoff[l] + slot * (pl.h[l] + P) * pl.astr[l]; };
  auto g_slot = [&](int l) { return lds + pl.goff[l] + slot * (pl.h[l] + P) * pl.gstr[l]; };
  // pointers to the top-left corner of the conv window of element (0,0) of the stack
  auto a_plane = [&](int l, int s) { return lds + pl.aoff[l] + s * pl.apl[l] + (P - R) * pl.astr[l] + (P - R); };
  auto g_plane = [&](int l, int s) { return lds + pl.goff[l] + s * pl.gpl[l]; };
  auto rows = [&](int l) { return pb * (pl.h[l] + P) - P; };

  const int b_begin = chunk * bchunk;
  const int b_end = b_begin + bchunk < B ? b_begin + bchunk : B;
  float xa[1][4], xb[1][4], ga[1][4], gb[1][4];
  if (pl.prefetch && has_slot) {
    const bool valid = b_begin + slot < b_end;
    const size_t off = (static_cast<size_t>(valid ? b_begin + slot : b_begin) * nC + c) * plane_elems;
    plane_fetch<T, 1>(x + off, pl.H, pl.W, ltid, nps, xa, xb);
    plane_fetch<T, 1>(g + off, pl.H, pl.W, ltid, nps, ga, gb);
  }
  zero_lds(lds, pl.lds_floats);          // while the first planes are on their way from HBM
  WT_LDS_BARRIER();

  for (int bv = b_begin; bv < b_end; bv += pb) {
    const int b0 = WT_UNIFORM(bv);
    WT_LAUNDER_LANE_INT(slot);
    WT_LAUNDER_LANE_INT(ltid);
    WT_LAUNDER_LANE_INT(lane);
    const bool valid = has_slot && b0 + slot < b_end;
    const size_t plane_off = (static_cast<size_t>(valid ? b0 + slot : b0) * nC + c) * plane_elems;
    int l0 = 2;
    WT_WAVE_PRIORITY(3);
    if (pl.prefetch && pl.fuse >= 2) {      // one plane per iteration: every lane takes part
      plane_commit_fused<1>(xa, xb, pl.H, pl.W, lds + pl.aoff[0], pl.astr[0], P, lds + pl.aoff[1], pl.astr[1],
                            pl.apl[1], lds + pl.aoff[2], pl.astr[2], pl.apl[2], lds + pl.aoff[pl.fuse],
                            pl.astr[pl.fuse], pl.apl[pl.fuse], P, pl.fuse, tid, blockDim.x);
      plane_commit_fused<1>(ga, gb, pl.H, pl.W, lds + pl.goff[0], pl.gstr[0], 0, lds + pl.goff[1], pl.gstr[1],
                            pl.gpl[1], lds + pl.goff[2], pl.gstr[2], pl.gpl[2], lds + pl.goff[pl.fuse],
                            pl.gstr[pl.fuse], pl.gpl[pl.fuse], 0, pl.fuse, tid, blockDim.x);
      l0 = pl.fuse + 1;
    } else if (pl.prefetch) {
      if (has_slot) {
        plane_commit<1>(xa, xb, pl.H, pl.W, a_slot(0), pl.astr[0], P, a_slot(1), pl.astr[1], pl.apl[1], P, ltid, nps,
                        valid);
        plane_commit<1>(ga, gb, pl.H, pl.W, g_slot(0), pl.gstr[0], 0, g_slot(1), pl.gstr[1], pl.gpl[1], 0, ltid, nps,
                        valid);
      }
    } else if (pl.vec_ok) {
      if (has_slot) {
        load_analysis1<T>(x + plane_off, pl.H, pl.W, a_slot(0), pl.astr[0], P, a_slot(1), pl.astr[1], pl.apl[1], P,
                          ltid, nps, valid);
        load_analysis1<T>(g + plane_off, pl.H, pl.W, g_slot(0), pl.gstr[0], 0, g_slot(1), pl.gstr[1], pl.gpl[1], 0,
                          ltid, nps, valid);
      }
    } else {
      if (has_slot) {
        load_plane<T>(x + plane_off, a_slot(0), pl.H, pl.W, pl.astr[0], P, ltid, nps, valid);
        load_plane<T>(g + plane_off, g_slot(0), pl.H, pl.W, pl.gstr[0], 0, ltid, nps, valid);
      }
      l0 = 1;
    }
    WT_LDS_BARRIER();
    if (pl.prefetch && has_slot && b0 + pb < b_end) {
      const bool nvalid = b0 + pb + slot < b_end;
      const size_t off = (static_cast<size_t>(nvalid ? b0 + pb + slot : b0) * nC + c) * plane_elems;
      plane_fetch<T, 1>(x + off, pl.H, pl.W, ltid, nps, xa, xb);   // an absent plane re-reads plane b0:
      plane_fetch<T, 1>(g + off, pl.H, pl.W, ltid, nps, ga, gb);   //   zeroed at commit
    }
    for (int lv = l0; lv <= L; ++lv) {
      const int l = WT_UNIFORM(lv);
      if (has_slot) {
        analysis_level(a_slot(l - 1), pl.astr[l - 1], P, a_slot(l), pl.astr[l], pl.apl[l], P, pl.h[l], pl.w[l],
                       ltid, nps);
        analysis_level(g_slot(l - 1), pl.gstr[l - 1], 0, g_slot(l), pl.gstr[l], pl.gpl[l], 0, pl.h[l], pl.w[l],
                       ltid, nps);
      }
      WT_LDS_BARRIER();
    }
    WT_WAVE_PRIORITY(0);
    // Both roles run the same code on different planes (one code path keeps a single
    // register set for the sums).
    {
      const int l = role_a ? 0 : 1;            // set 0, strips of TJ: base conv rows (A) / level 1 (B)
      corr_level<K, TJ, VW, true>(a_plane(l, role_a ? 0 : q), pl.astr[l], g_plane(l, role_a ? 0 : q), pl.gstr[l],
                            rows(l), pl.w[l], lane, role_a ? q : 0, role_a ? 4 : 1, acc[0]);
    }
    if (wave == 0) {
      // bias gradient: the sum of grad_out is 2^L times the sum of its coarsest LL band (every
      // Haar level halves the sum of a plane; padding, gap rows and absent planes hold zeros)
      const float* GL = g_plane(L, 0);
      const int n = imul(rows(L), pl.gstr[L]);
      for (int e = lane; e < n; e += kWave) gsum += GL[e];
    }
    if constexpr (NSET >= 2) {                 // set 1, single coefficients: level 3 (A) / level 2 (B)
      const int l = role_a ? 3 : 2;
      if (l <= L) {
        // a level at least kStripMinWidth wide is walked in row pairs of TJ-wide strips like the
        // first set (one pass of a wave instead of four at 14 x 14), a narrower one by single
        // coefficients (more lanes busy)
        if (pl.w[l] >= kStripMinWidth)
          corr_level<K, TJ, VW, true>(a_plane(l, q), pl.astr[l], g_plane(l, q), pl.gstr[l], rows(l), pl.w[l], lane, 0,
                                      1, acc[1]);
        else
          corr_level<K, 1, 1, false>(a_plane(l, q), pl.astr[l], g_plane(l, q), pl.gstr[l], rows(l), pl.w[l], lane, 0,
                                     1, acc[1]);
      }
    }
    if constexpr (NSET >= 3) {                 // set 2: level 5 (A) / level 4 (B)
      const int l = role_a ? 5 : 4;
      if (l <= L) {
        corr_level<K, 1, 1, false>(a_plane(l, q), pl.astr[l], g_plane(l, q), pl.gstr[l], rows(l), pl.w[l], lane, 0, 1,
                                   acc[2]);
      }
    }
    WT_LDS_BARRIER();
  }

  // cross-lane reduction, then cross-wave through LDS (pyramid buffers are dead now)
  constexpr int NRED = NSET * KK + 1;
  float* red = lds;   // [8 waves][NRED]
#pragma unroll
  for (int s = 0; s < NSET; ++s)
#pragma unroll
    for (int t = 0; t < KK; ++t) {
      const float v = wave_sum(acc[s][t]);
      if (lane == 0) red[wave * NRED + s * KK + t] = v;
    }
  {
    const float v = wave_sum(gsum) * static_cast<float>(1 << L);
    if (lane == 0) red[wave * NRED + NRED - 1] = v;
  }
  WT_LDS_BARRIER();
  float* dst = partial + (static_cast<size_t>(chunk) * nC + c) * (NF * KK + 1);
  for (int o = tid; o < NF * KK + 1; o += blockDim.x) {
    float v = 0.f;
    if (o == NF * KK) {
      for (int wv = 0; wv < 4; ++wv) v += red[wv * NRED + NRED - 1];
    } else {
      const int f = o / KK, t = o - f * KK;
      if (f == 0) {
        for (int wv = 0; wv < 4; ++wv) v += red[wv * NRED + t];
      } else {
        const int l = 1 + ((f - 1) >> 2), s = (f - 1) & 3;
        // level -> (role, set): 1 -> B0, 2 -> B1, 3 -> A1, 4 -> B2, 5 -> A2
        const bool in_a = (l == 3) || (l == 5);
        const int set = l == 1 ? 0 : (l <= 3 ? 1 : 2);
        v = red[(in_a ? s : 4 + s) * NRED + set * KK + t];
      }
    }
    if (fin.tickets != nullptr) store_shared_f32(dst + o, v);
    else dst[o] = v;
  }
  wgrad_finish_if_last(fin, partial, static_cast<int>(gridDim.y), nC, c, 4, L, KK, lds);
}

// The second stage as a launch of its own (one workgroup per channel, dynamic LDS NF*KK + 1 floats): after a first
// stage that does not finish its channels itself.
__global__ void wgrad_finish_kernel(const float* __restrict__ partial, int nchunk, ParamTable p,
                                    int pdtype, GradTable gt, int C, int S, int L, int KK) {
  WT_SHARED_FLOATS(prod);
  wgrad_finish_channel<false>(partial, nchunk, p, pdtype, gt, C, static_cast<int>(blockIdx.x), S, L, KK, prod);
}

// Clears the ticket words of a first stage that finishes its channels itself (a kernel rather than a memset, so
// that a caller may record the call into a HIP graph).
__global__ void zero_tickets_kernel(unsigned* __restrict__ t, int n) {
  for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) t[i] = 0u;
}

}  // namespace wt
