// Host stand-in for the few HIP device facilities the WTConv kernels use, so that the
// kernel sources can be compiled with g++ and run under AddressSanitizer without a GPU.
// Test infrastructure only: a workgroup becomes a set of std::threads that meet at a
// barrier for __syncthreads(); LDS becomes an exactly-sized heap block so that any
// out-of-range LDS access is reported.
#pragma once

#include <barrier>
#include <cmath>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <memory>
#include <thread>
#include <vector>

#define __global__
#define __device__
#define __host__
#define __forceinline__ inline
#define __launch_bounds__(...)
#define __align__(n)
// workgroups run one after the other here: a function-local static is shared by exactly the
// threads of the running workgroup
#define __shared__ static

struct dim3 {
  unsigned x, y, z;
  dim3(unsigned x_ = 1, unsigned y_ = 1, unsigned z_ = 1) : x(x_), y(y_), z(z_) {}
};
struct uint2 { uint32_t x, y; };
struct alignas(16) uint4 { uint32_t x, y, z, w; };
struct float2 { float x, y; };
struct alignas(16) float4 { float x, y, z, w; };

typedef void* hipStream_t;

namespace emu {
struct BlockState {
  std::unique_ptr<std::barrier<>> bar;
  std::vector<std::unique_ptr<std::barrier<>>> wave_bar;   // one per wavefront of 64 threads
  float* lds = nullptr;
  std::vector<float> xchg;
  std::vector<uint16_t> mfma_a, mfma_b;                   // [thread][8] operand exchange of the emulated MFMA
  unsigned nthreads = 0;
};
inline thread_local BlockState* tls_block = nullptr;
inline float* lds_base() { return tls_block->lds; }
}  // namespace emu

inline thread_local dim3 threadIdx, blockIdx, blockDim, gridDim;

inline void __syncthreads() { emu::tls_block->bar->arrive_and_wait(); }

inline float __uint_as_float(uint32_t u) { float f; std::memcpy(&f, &u, 4); return f; }
inline uint32_t __float_as_uint(float f) { uint32_t u; std::memcpy(&u, &f, 4); return u; }

namespace emu {
// Barrier over the 64 threads of the calling thread's wavefront.
inline void wave_barrier() { tls_block->wave_bar[threadIdx.x / 64]->arrive_and_wait(); }
}  // namespace emu

// Every thread of the wavefront must call this the same number of times (true for the kernels here: reductions sit
// outside divergent code).  Lanes exchange within their wavefront only (mask < 64), so its barrier is enough.
inline float __shfl_xor(float v, int mask, int /*width*/) {
  emu::BlockState* b = emu::tls_block;
  b->xchg[threadIdx.x] = v;
  emu::wave_barrier();
  const float r = b->xchg[threadIdx.x ^ static_cast<unsigned>(mask)];
  emu::wave_barrier();
  return r;
}

namespace emu {

// D = A (16x32) * B (32x16) + C on bfloat16 operands with float accumulation, operands and
// result distributed over the 64 lanes of a wavefront as v_mfma_f32_16x16x32_bf16 holds them:
// lane l carries A[l % 16][8 * (l / 16) + j], B[8 * (l / 16) + j][l % 16] (j = 0..7) and
// D[4 * (l / 16) + r][l % 16] (r = 0..3).  Every lane of the wavefront must call it.
inline void mfma_16x16x32_bf16(const uint16_t (&a)[8], const uint16_t (&b)[8], float (&c)[4]) {
  BlockState* st = tls_block;
  const unsigned t = threadIdx.x, wbase = t / 64 * 64, l = t % 64;
  for (int j = 0; j < 8; ++j) { st->mfma_a[t * 8 + j] = a[j]; st->mfma_b[t * 8 + j] = b[j]; }
  wave_barrier();
  auto f = [](uint16_t v) { uint32_t u = static_cast<uint32_t>(v) << 16; float x; std::memcpy(&x, &u, 4); return x; };
  const unsigned n = l % 16, q = l / 16;
  for (int r = 0; r < 4; ++r) {
    const unsigned m = 4 * q + r;
    float acc = c[r];
    for (unsigned kq = 0; kq < 4; ++kq)
      for (int j = 0; j < 8; ++j)
        acc += f(st->mfma_a[(wbase + 16 * kq + m) * 8 + j]) * f(st->mfma_b[(wbase + 16 * kq + n) * 8 + j]);
    c[r] = acc;
  }
  wave_barrier();
}

template <typename F>
void launch(dim3 grid, dim3 block, size_t lds_bytes, F body) {
  const unsigned nt = block.x * block.y * block.z;
  for (unsigned bz = 0; bz < grid.z; ++bz)
    for (unsigned by = 0; by < grid.y; ++by)
      for (unsigned bx = 0; bx < grid.x; ++bx) {
        BlockState st;
        st.bar = std::make_unique<std::barrier<>>(nt);
        st.nthreads = nt;
        st.xchg.assign(nt, 0.f);
        st.mfma_a.assign(static_cast<size_t>(nt) * 8, 0);
        st.mfma_b.assign(static_cast<size_t>(nt) * 8, 0);
        for (unsigned wv = 0; wv < (nt + 63) / 64; ++wv) {
          const unsigned in_wave = nt - wv * 64 < 64 ? nt - wv * 64 : 64;
          st.wave_bar.push_back(std::make_unique<std::barrier<>>(in_wave));
        }
        // exact size: ASan red zones catch LDS overruns; filled with NaN so that reads of
        // never-written LDS show up in results
        float* lds = lds_bytes ? static_cast<float*>(std::aligned_alloc(16, (lds_bytes + 15) / 16 * 16)) : nullptr;
        for (size_t i = 0; i < lds_bytes / 4; ++i) lds[i] = std::nanf("");
        st.lds = lds;
        std::vector<std::thread> th;
        th.reserve(nt);
        for (unsigned t = 0; t < nt; ++t) {
          th.emplace_back([&, t]() {
            tls_block = &st;
            threadIdx = dim3(t % block.x, (t / block.x) % block.y, t / (block.x * block.y));
            blockIdx = dim3(bx, by, bz);
            blockDim = block;
            gridDim = grid;
            body();
          });
        }
        for (auto& x : th) x.join();
        std::free(lds);
      }
}
}  // namespace emu

inline int __clz(int v) { return v == 0 ? 32 : __builtin_clz(static_cast<unsigned>(v)); }
