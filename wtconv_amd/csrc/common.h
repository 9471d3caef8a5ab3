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
#include <type_traits>

#include "../../include/wtconv_hip.h"

#ifdef WT_EMULATE
#define WT_SHARED_FLOATS(name) float* name = ::emu::lds_base()
#define WT_SCHED_FENCE() do {} while (0)
#define WT_UNIFORM(x) (x)
#define WT_LDS_BARRIER() __syncthreads()
#define WT_WAVE_LDS_SYNC() __syncthreads()
#define WT_WAIT_VMEM() do {} while (0)
#define WT_CHUNK_FENCE() do {} while (0)
#define WT_LAUNDER_UNIFORM_PTR(p) do {} while (0)
#define WT_LAUNDER_LANE_INT(v) do {} while (0)
#define WT_WAVE_PRIORITY(n) do {} while (0)
typedef const float* wt_uniform_ptr;
#else
// Folded weights are read-only for the whole launch and indexed uniformly: the constant
// address space makes the compiler fetch them with scalar loads into SGPRs even after a
// barrier (global-address-space loads fall back to per-lane vector loads there).
typedef const float __attribute__((address_space(4)))* wt_uniform_ptr;
#define WT_SHARED_FLOATS(name) extern __shared__ __align__(16) float name[]
// nothing may be scheduled across this point (keeps LDS reads from being hoisted en masse)
#define WT_SCHED_FENCE() __builtin_amdgcn_sched_barrier(0)
// tells the compiler that an int is the same in every lane (keeps it in an SGPR, so that
// everything indexed by it is fetched with scalar loads)
#define WT_UNIFORM(x) __builtin_amdgcn_readfirstlane(x)
// Workgroup barrier that orders LDS traffic only.  __syncthreads() would also wait for
// every outstanding HBM load, i.e. for the prefetch of the next plane issued just before.
#define WT_LDS_BARRIER()                                                \
  do {                                                                  \
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");     \
    __builtin_amdgcn_s_barrier();                                       \
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");     \
  } while (0)
// Orders the LDS traffic of one wave only: lanes of a wave that exchange data through LDS (a
// plane owned by 64 lanes or fewer) need no workgroup barrier, because the LDS instructions of a
// wave execute in issue order; this only keeps the compiler from moving them across.
#define WT_WAVE_LDS_SYNC()                                              \
  do {                                                                  \
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront", "local");     \
    __builtin_amdgcn_wave_barrier();                                    \
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront", "local");     \
  } while (0)
// s_waitcnt vmcnt(0) only (gfx9 encoding: expcnt and lgkmcnt left at their maxima).
// gfx950 counts loads and stores in the same counter; waiting for the prefetch loads
// *before* the output stores are issued lets those stores drain in the background instead
// of being waited for at the top of the next plane.
#define WT_WAIT_VMEM() __builtin_amdgcn_s_waitcnt(0x0F70)
// Compiler-level fence between the chunks of a work item: memory operations (the LDS row
// reads of the next chunk) may not be moved above it, which bounds the live registers to
// one chunk's rows.  Emits no instruction.
#define WT_CHUNK_FENCE() do { asm volatile("" ::: "memory"); __builtin_amdgcn_sched_barrier(0); } while (0)
// Makes a uniform pointer opaque at this point, so that the scalar weight loads behind it
// are issued here (25 SGPRs live) instead of being hoisted out of the row loop all at once
// (hundreds of SGPRs, spilled to VGPR lanes).
#define WT_LAUNDER_UNIFORM_PTR(p) asm volatile("" : "+s"(p))
// Makes a per-lane index opaque inside a loop body, so that the addresses derived from it
// are recomputed per iteration (a few integer ops) instead of being hoisted out of the loop
// into long-lived registers that end up spilled.
#define WT_LAUNDER_LANE_INT(v) asm volatile("" : "+v"(v))
// Issue priority of this wave against the other waves of its SIMD (0 = default, 3 = highest).
// The short serial phases of a plane (few work items, barrier after barrier) run at high
// priority so that they are not slowed down to a quarter of their speed by the arithmetic-heavy
// phases of the other workgroups on the same SIMD, which fill whatever issue slots are left.
#define WT_WAVE_PRIORITY(n) __builtin_amdgcn_s_setprio(n)
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

// round-to-nearest-even, NaN kept quiet.  On the device this is the hardware conversion
// (v_cvt_pk_bf16_f32, one instruction per two values); the host emulation spells it out.
#ifdef WT_EMULATE
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return static_cast<bf16_t>((u >> 16) | 0x40u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return static_cast<bf16_t>(u >> 16);
}
// two values in one 32-bit word, `lo` in the low half
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  return static_cast<uint32_t>(f32_to_bf16(lo)) | (static_cast<uint32_t>(f32_to_bf16(hi)) << 16);
}
#else
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
  return __builtin_bit_cast(bf16_t, static_cast<__bf16>(f));
}
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  typedef float wt_f32x2 __attribute__((ext_vector_type(2)));
  typedef __bf16 wt_bf16x2 __attribute__((ext_vector_type(2)));
  const wt_f32x2 v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, wt_bf16x2));
}
#endif

// IEEE half storage: a type of its own, so that templates tell it from bf16.  The vector-ALU kernels read and write
// it and compute in fp32 (haar_common.cuh:55-77 of the reference dispatches the same three element types).
struct f16_t { uint16_t bits; };

#ifdef WT_EMULATE
__device__ __forceinline__ float f16_bits_to_f32(uint16_t h) {
  const uint32_t sign = static_cast<uint32_t>(h & 0x8000u) << 16;
  const uint32_t ex = (h >> 10) & 31u, man = h & 0x3ffu;
  if (ex == 31u) return __uint_as_float(sign | 0x7f800000u | (man << 13));
  if (ex == 0u) {                                        // zero and subnormals: man * 2^-24, exact in fp32
    const float v = static_cast<float>(man) * 5.9604644775390625e-8f;
    return sign ? -v : v;
  }
  return __uint_as_float(sign | ((ex + 112u) << 23) | (man << 13));
}
// round-to-nearest-even, overflow to infinity, NaN kept quiet
__device__ __forceinline__ uint16_t f32_to_f16_bits(float f) {
  const uint32_t u = __float_as_uint(f);
  const uint16_t sign = static_cast<uint16_t>((u >> 16) & 0x8000u);
  const uint32_t a = u & 0x7fffffffu;
  if (a > 0x7f800000u) return static_cast<uint16_t>(sign | 0x7e00u);
  if (a >= 0x477ff000u) return static_cast<uint16_t>(sign | 0x7c00u);      // >= 65520 rounds to infinity
  if (a < 0x33000001u) return sign;                                        // <= 2^-25 rounds to zero
  const int e = static_cast<int>(a >> 23) - 127;
  uint32_t man = (a & 0x7fffffu) | 0x800000u;                              // 24 significant bits
  const int shift = e >= -14 ? 13 : 13 + (-14 - e);                        // bits dropped (subnormals drop more)
  const uint32_t kept = man >> shift, rest = man & ((1u << shift) - 1u), half = 1u << (shift - 1);
  uint32_t r = kept + ((rest > half || (rest == half && (kept & 1u))) ? 1u : 0u);
  // normal: r holds the implicit one at bit 10, so adding the biased exponent - 1 carries correctly on mantissa overflow
  const uint32_t bits = e >= -14 ? (static_cast<uint32_t>(e + 14) << 10) + r : r;
  return static_cast<uint16_t>(sign | bits);
}
#else
__device__ __forceinline__ float f16_bits_to_f32(uint16_t h) {
  return static_cast<float>(__builtin_bit_cast(_Float16, h));
}
__device__ __forceinline__ uint16_t f32_to_f16_bits(float f) {
  return __builtin_bit_cast(uint16_t, static_cast<_Float16>(f));
}
#endif

template <typename T> __device__ __forceinline__ float to_f32(T v);
template <> __device__ __forceinline__ float to_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ float to_f32<bf16_t>(bf16_t v) { return bf16_to_f32(v); }
template <> __device__ __forceinline__ float to_f32<f16_t>(f16_t v) { return f16_bits_to_f32(v.bits); }

template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16_t from_f32<bf16_t>(float v) { return f32_to_bf16(v); }
template <> __device__ __forceinline__ f16_t from_f32<f16_t>(float v) { return f16_t{f32_to_f16_bits(v)}; }

// Two 16-bit elements of type T in one 32-bit word (the first in the low half): unpack to fp32, pack from fp32.
template <typename T> __device__ __forceinline__ void unpack2(uint32_t w, float& lo, float& hi);
template <> __device__ __forceinline__ void unpack2<bf16_t>(uint32_t w, float& lo, float& hi) {
  lo = __uint_as_float(w << 16); hi = __uint_as_float(w & 0xffff0000u);
}
template <> __device__ __forceinline__ void unpack2<f16_t>(uint32_t w, float& lo, float& hi) {
  lo = f16_bits_to_f32(static_cast<uint16_t>(w)); hi = f16_bits_to_f32(static_cast<uint16_t>(w >> 16));
}
template <typename T> __device__ __forceinline__ uint32_t pack2(float lo, float hi);
template <> __device__ __forceinline__ uint32_t pack2<bf16_t>(float lo, float hi) { return pack_bf16x2(lo, hi); }
template <> __device__ __forceinline__ uint32_t pack2<f16_t>(float lo, float hi) {
#ifdef WT_EMULATE
  return static_cast<uint32_t>(f32_to_f16_bits(lo)) | (static_cast<uint32_t>(f32_to_f16_bits(hi)) << 16);
#else
  typedef float wt_f32x2 __attribute__((ext_vector_type(2)));
  typedef _Float16 wt_f16x2 __attribute__((ext_vector_type(2)));
  const wt_f32x2 v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, wt_f16x2));
#endif
}

// parameter fetch with a run-time dtype (only used while folding parameters)
__device__ __forceinline__ float load_param(const void* p, int dtype, int idx) {
  if (dtype == WTCONV_F32) return static_cast<const float*>(p)[idx];
  const uint16_t h = static_cast<const uint16_t*>(p)[idx];
  return dtype == WTCONV_F16 ? f16_bits_to_f32(h) : bf16_to_f32(h);
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

// Value of lane `src` (a constant) of the calling wavefront, as a wave-uniform value (v_readlane_b32: the result lives
// in an SGPR, so an FMA takes it as its scalar operand).  The host emulation has no lanes to read from: there every
// thread holds the whole table and indexes it itself (see LaneTable).
#ifndef WT_EMULATE
__device__ __forceinline__ float lane_bcast(float v, int src) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), src));
}
#endif

// N wave-uniform floats kept one per lane: entry i in lane i % 64 of word i / 64 of every wavefront (N / 64 vector
// registers instead of N; reading entry i costs one v_readlane).  This is how the vector-ALU kernels hold the
// folded parameters of their channel when they fold them themselves.
template <int N>
struct LaneTable {
#ifdef WT_EMULATE
  float v[N];
  __device__ __forceinline__ float get(int i) const { return v[i]; }
  template <typename F> __device__ __forceinline__ void fill(F&& f) {
    for (int i = 0; i < N; ++i) v[i] = f(i);
  }
#else
  static constexpr int kWords = (N + kWave - 1) / kWave;
  float v[kWords];
  // `i` must be a compile-time constant after unrolling (v_readlane takes the lane as an immediate or an SGPR)
  __device__ __forceinline__ float get(int i) const { return lane_bcast(v[i / kWave], i % kWave); }
  // f(i) is evaluated by the lane that keeps entry i
  template <typename F> __device__ __forceinline__ void fill(F&& f) {
    const int lane = static_cast<int>(threadIdx.x) & (kWave - 1);
#pragma unroll
    for (int j = 0; j < kWords; ++j) {
      const int i = lane + j * kWave;
      v[j] = i < N ? f(i) : 0.f;
    }
  }
#endif
};

// Hand-over between the workgroups of one launch.  What a workgroup leaves for another one to read (its record of
// partial sums) is stored with store_shared_f32 and read with load_shared_f32: device-scope accesses that go through
// to / come from the memory all compute units see, whichever L2 the two workgroups sit behind.  No cache is written
// back or invalidated as a whole (a device-scope fence would do that once per workgroup, and every one of them would
// have to go through everything the launch has written so far).
#ifdef WT_EMULATE
__device__ __forceinline__ void store_shared_f32(float* p, float v) { *p = v; }
__device__ __forceinline__ float load_shared_f32(const float* p) { return *p; }
#else
__device__ __forceinline__ void store_shared_f32(float* p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float load_shared_f32(const float* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
#endif

// Every thread calls this after its store_shared_f32 stores: they are waited for, one ticket is drawn, and the call
// returns true in the workgroup that drew the last of `total` (the same value in all its threads), which may then
// read with load_shared_f32 what every other workgroup stored before its own call.  `flag` = one word of LDS.  The
// ticket word must be zero when the launch starts; the last workgroup leaves it zero again.
__device__ __forceinline__ bool workgroup_is_last(unsigned* __restrict__ ticket, unsigned total, unsigned* flag) {
#ifdef WT_EMULATE
  __syncthreads();
  if (threadIdx.x == 0) { *flag = (*ticket == total - 1) ? 1u : 0u; *ticket += 1u; }   // (workgroups run one after the other)
  __syncthreads();
  return *flag != 0u;
#else
  __builtin_amdgcn_s_waitcnt(0x0F70);      // vmcnt(0): this thread's stores have been acknowledged
  __syncthreads();
  if (threadIdx.x == 0)
    *flag = __hip_atomic_fetch_add(ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == total - 1 ? 1u : 0u;
  __syncthreads();
  return *flag != 0u;
#endif
}

// Orders the computation of v[] before the next WT_CHUNK_FENCE (the fence alone only
// orders memory operations; arithmetic would otherwise be sunk below it and every row read
// of a work item would stay live at once).  Emits no instruction.
template <int N>
__device__ __forceinline__ void pin_values(float (&v)[N]) {
#ifndef WT_EMULATE
#pragma unroll
  for (int i = 0; i < N; ++i) asm volatile("" : "+v"(v[i]));
#else
  (void)v;
#endif
}

// 16-byte global accesses of data that is touched once (activations streaming through a kernel): marked
// non-temporal, so that they do not displace what the caches should keep.
__device__ __forceinline__ uint4 load_stream_u4(const void* p) {
#ifdef WT_EMULATE
  return *reinterpret_cast<const uint4*>(p);
#else
  typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
  const u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(p));
  uint4 r;
  r.x = v.x; r.y = v.y; r.z = v.z; r.w = v.w;
  return r;
#endif
}
__device__ __forceinline__ void store_stream_u4(void* p, const uint4& q) {
#ifdef WT_EMULATE
  *reinterpret_cast<uint4*>(p) = q;
#else
  typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
  u32x4_t v;
  v.x = q.x; v.y = q.y; v.z = q.z; v.w = q.w;
  __builtin_nontemporal_store(v, reinterpret_cast<u32x4_t*>(p));
#endif
}

// Workgroups of a launch are dealt to the eight XCDs of the GPU in turn (workgroup i runs on XCD i % 8, each with an
// L2 of its own).  Index i of n -> an index such that the workgroups of one XCD hold a contiguous range, neighbours in
// it being dispatched next to each other: planes that share cache lines (small planes of adjacent channels) then meet
// in one L2.  A bijection on [0, n); the identity when n is no multiple of 8.
__device__ __forceinline__ int xcd_contiguous(int i, int n) {
  return (n & 7) == 0 ? (i & 7) * (n >> 3) + (i >> 3) : i;
}

// Product of two indices that fit 24 bits (rows, strides and offsets inside a plane or the
// LDS): v_mul_i32_i24 runs at full rate, the 32-bit v_mul_lo_u32 at a quarter of it.
__device__ __forceinline__ int imul(int a, int b) {
#ifdef WT_EMULATE
  return a * b;
#else
  return __mul24(a, b);
#endif
}

// Value of lane (lane ^ mask) of the wavefront; `lane4` = 4 * lane, computed once by the
// caller, so that one exchange costs one integer op and one ds_bpermute (the generic
// __shfl_xor recomputes and range-checks the source lane every time).
__device__ __forceinline__ float wave_xor(float v, int lane4, int mask) {
#ifdef WT_EMULATE
  (void)lane4;
  return __shfl_xor(v, mask, kWave);
#else
  return __int_as_float(__builtin_amdgcn_ds_bpermute(lane4 ^ (mask << 2), __float_as_int(v)));
#endif
}

// Sum over the 64 lanes of a wavefront; every lane gets the total.  On the GPU: six DPP adds
// (quad permutes, row mirrors, row broadcasts) and one v_readlane, no LDS traffic -- the
// weight-gradient kernels reduce up to 76 running sums per workgroup this way.
__device__ __forceinline__ float wave_sum(float v) {
#ifdef WT_EMULATE
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m, kWave);
  return v;
#else
  auto dpp = [](float x, auto ctrl, auto row_mask) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), decltype(ctrl)::value,
                                                      decltype(row_mask)::value, 0xf, false));
  };
  using std::integral_constant;
  v += dpp(v, integral_constant<int, 0xB1>{}, integral_constant<int, 0xf>{});    // quad_perm [1,0,3,2]
  v += dpp(v, integral_constant<int, 0x4E>{}, integral_constant<int, 0xf>{});    // quad_perm [2,3,0,1]
  v += dpp(v, integral_constant<int, 0x141>{}, integral_constant<int, 0xf>{});   // row_half_mirror
  v += dpp(v, integral_constant<int, 0x140>{}, integral_constant<int, 0xf>{});   // row_mirror: row sums
  v += dpp(v, integral_constant<int, 0x142>{}, integral_constant<int, 0xa>{});   // row_bcast:15 into rows 1, 3
  v += dpp(v, integral_constant<int, 0x143>{}, integral_constant<int, 0xc>{});   // row_bcast:31 into rows 2, 3
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
#endif
}

}  // namespace wt
