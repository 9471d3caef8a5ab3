// Second stage of the parameter gradients, as a device function: shared by the kernel that runs it as a launch of
// its own and by the first-stage kernels that finish their channels themselves (the workgroup that completes a
// channel last runs it for that channel).
#pragma once

#include "common.h"

namespace wt {

// Second stage: sum the per-chunk partials and apply the chain rule of the folding
//   dw = gamma * dWt,  dgamma = sum_t w * dWt (+ bias * sumG for the base scale),
//   dbias = gamma_b * sumG        (cf. fast_wtconv/cuda_haar/haar_cuda.py:168-197,657-676)
// for one channel, by the threads of one workgroup: one thread per (filter, tap) plus one for sumG where the
// workgroup has that many (else strided); the per-filter dot products go through `prod` (NF*KK + 1 floats of
// LDS).  S = 4 (2-D) or 2 (1-D).  blockDim.x >= NF.  The chunks are summed in index order whichever workgroup
// runs this, so the result does not depend on the order in which the first stage finished.  SHARED: called by the
// last workgroup of a first stage that finishes its channels itself: the records of the other workgroups are read
// with load_shared_f32.
template <bool SHARED>
__device__ __forceinline__ void wgrad_finish_channel(const float* __restrict__ partial, int nchunk,
                                                     const ParamTable& p, int pdtype, const GradTable& gt, int C,
                                                     int c, int S, int L, int KK, float* __restrict__ prod) {
  const int NF = 1 + S * L;
  const int stride = NF * KK + 1;
  // table entries of a level picked with constant indices (a per-lane index into the argument structs would send
  // them to scratch memory)
  auto level_w = [&](int l) { const void* q = p.wt_weight[0];
#pragma unroll
    for (int i = 1; i < kMaxLevels; ++i) q = l == i ? p.wt_weight[i] : q; return q; };
  auto level_s = [&](int l) { const void* q = p.wt_scale[0];
#pragma unroll
    for (int i = 1; i < kMaxLevels; ++i) q = l == i ? p.wt_scale[i] : q; return q; };
  auto grad_w = [&](int l) { float* q = gt.wt_weight[0];
#pragma unroll
    for (int i = 1; i < kMaxLevels; ++i) q = l == i ? gt.wt_weight[i] : q; return q; };
  auto grad_s = [&](int l) { float* q = gt.wt_scale[0];
#pragma unroll
    for (int i = 1; i < kMaxLevels; ++i) q = l == i ? gt.wt_scale[i] : q; return q; };
  for (int o = threadIdx.x; o <= NF * KK; o += blockDim.x) {      // (the last index is the sumG slot of the records)
    const bool tap = o < NF * KK;
    const int f = tap ? o / KK : 0, t = tap ? o - f * KK : 0;
    const int l = f == 0 ? 0 : (f - 1) / S, chn = f == 0 ? c : c * S + (f - 1) % S;
    // parameters first: their loads overlap those of the partial sums
    const float gam = load_param(f == 0 ? p.base_scale : level_s(l), pdtype, chn);
    const float wv = load_param(f == 0 ? p.base_weight : level_w(l), pdtype, chn * KK + t);
    float sum = 0.f;
#pragma unroll 8                       // several chunk loads in flight; the order of the adds is unchanged
    for (int ch = 0; ch < nchunk; ++ch) {
      const float* src = partial + (static_cast<size_t>(ch) * C + c) * stride + o;
      sum += SHARED ? load_shared_f32(src) : *src;
    }
    if (tap) {
      float* dst = f == 0 ? gt.base_weight : grad_w(l);
      dst[chn * KK + t] = gam * sum;
      prod[o] = wv * sum;
    } else {
      prod[o] = sum;
    }
  }
  const int o = threadIdx.x;
  __syncthreads();
  if (o < NF) {
    float dot = 0.f;
    for (int t = 0; t < KK; ++t) dot += prod[o * KK + t];
    if (o == 0) {
      const float sg = prod[NF * KK];
      if (p.base_bias != nullptr) {
        dot = fmaf(load_param(p.base_bias, pdtype, c), sg, dot);
        if (gt.base_bias != nullptr) gt.base_bias[c] = load_param(p.base_scale, pdtype, c) * sg;
      }
      gt.base_scale[c] = dot;
    } else {
      const int l = (o - 1) / S, chn = c * S + (o - 1) % S;
      grad_s(l)[chn] = dot;
    }
  }
}

// What a first-stage kernel needs to finish its channels itself.  tickets == nullptr: it only stores its records and
// wgrad_finish_kernel runs afterwards.  Otherwise `tickets` holds one zero word per channel.
struct FinishArgs {
  unsigned* tickets;
  ParamTable prm;
  int pdtype;
  GradTable gt;
};

// End of a first-stage workgroup (channel c, `nchunk` workgroups per channel, records of `nrec` floats stored with
// store_shared_f32 when fin.tickets is set): draws the channel's ticket and, in the last workgroup, runs the second
// stage.  `lds`: at least nrec + 1 floats that no thread still reads from before its call.
__device__ __forceinline__ void wgrad_finish_if_last(const FinishArgs& fin, const float* __restrict__ partial,
                                                     int nchunk, int C, int c, int S, int L, int KK,
                                                     float* __restrict__ lds) {
  if (fin.tickets == nullptr) return;
  const int nrec = (1 + S * L) * KK + 1;
  unsigned* flag = reinterpret_cast<unsigned*>(lds + nrec);
  if (workgroup_is_last(fin.tickets + c, static_cast<unsigned>(nchunk), flag)) {
    wgrad_finish_channel<true>(partial, nchunk, fin.prm, fin.pdtype, fin.gt, C, c, S, L, KK, lds);
    if (threadIdx.x == 0) fin.tickets[c] = 0u;
  }
}

}  // namespace wt
