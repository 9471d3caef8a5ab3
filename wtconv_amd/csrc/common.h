// Shared device/host helpers for the WTConv gfx950 kernels.
//
// The kernel sources compile two ways: with hipcc for gfx950 (the product), and with a
// plain host compiler when WT_EMULATE is defined, in which case "emu_runtime.h" (under
// tests/) supplies threadIdx/__syncthreads/__shfl_xor on top of std::thread so that the
// indexing of every kernel can be run under AddressSanitizer on a machine without a GPU.
#pragma once

#ifdef WT_EMULATE
#include "emu_runtime.h"
#else
#include <hip/hip_runtime.h>
#endif
#include <stdint.h>

#include "../../include/wtconv_hip.h"

#ifdef WT_EMULATE
#define WT_SHARED_FLOATS(name) float* name = ::emu::lds_base()
#else
#define WT_SHARED_FLOATS(name) extern __shared__ __align__(16) float name[]
#endif

namespace wt {

constexpr int kMaxLevels = WTCONV_MAX_LEVELS;
constexpr int kWave = 64;                   // CDNA wavefront
constexpr int kLdsLimitBytes = 160 * 1024;  // LDS per CU on gfx950
constexpr int kLdsSlackFloats = 64;         // strips may read a few floats past a row end

typedef uint16_t bf16_t;                    // raw bfloat16 storage

__device__ __forceinline__ float bf16_to_f32(bf16_t v) {
  return __uint_as_float(static_cast<uint32_t>(v) << 16);
}

// round-to-nearest-even, NaN kept quiet
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return static_cast<bf16_t>((u >> 16) | 0x40u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return static_cast<bf16_t>(u >> 16);
}

template <typename T> __device__ __forceinline__ float to_f32(T v);
template <> __device__ __forceinline__ float to_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ float to_f32<bf16_t>(bf16_t v) { return bf16_to_f32(v); }

template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16_t from_f32<bf16_t>(float v) { return f32_to_bf16(v); }

// parameter fetch with a run-time dtype (only used while folding parameters)
__device__ __forceinline__ float load_param(const void* p, int dtype, int idx) {
  return dtype == WTCONV_F32 ? static_cast<const float*>(p)[idx]
                             : bf16_to_f32(static_cast<const bf16_t*>(p)[idx]);
}

// Kernel-argument copy of wtconv_params.
struct ParamTable {
  const void* base_weight;
  const void* base_bias;
  const void* base_scale;
  const void* wt_weight[kMaxLevels];
  const void* wt_scale[kMaxLevels];
};

struct GradTable {
  float* base_weight;
  float* base_bias;
  float* base_scale;
  float* wt_weight[kMaxLevels];
  float* wt_scale[kMaxLevels];
};

// Sum over the 64 lanes of a wavefront; every lane gets the total.
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m, kWave);
  return v;
}

}  // namespace wt
