// Row-resident WTConv1d kernels for gfx950.
//
// One workgroup owns a whole (b, c) row; every lane owns S consecutive samples and keeps
// them, their complete Haar pyramid and the outputs in registers.  S is a multiple of 2^L, so
// the analysis and synthesis butterflies never leave the lane.  The K-tap conv of a level
// needs R = K/2 coefficients from beyond either end of the lane's array: each lane publishes
// the edge entries of each of its arrays in LDS once per row, and reads its neighbours'
// (on the coarsest levels, where a lane holds fewer than R coefficients, from up to R lanes
// away).  LDS is otherwise used only to turn coalesced 16-byte HBM accesses into the
// lane-contiguous register layout and back (slot stride = odd number of 16-byte units:
// conflict-free both ways).  Three workgroup barriers per row instead of one per pyramid
// level and phase.
//
// Maths as in kernels1d.h (reference wtconv/wtconv1d.py:38-82, wtconv/util/wavelet.py:6-20,
// 46-59).  Samples past the end of the row are staged as zeros, which gives the 'same'
// padding of every level and the zero padding of odd lengths at once.
#pragma once

#include "common.h"
#include "kernels1d.h"

namespace wt {

// Samples per lane: a multiple of 2^L (the pyramid of a lane is local) and of 8 (16-byte
// vectors of either dtype).  32 from four levels on (measured faster than 16 at L = 4: fewer
// edge exchanges per sample), 16 below.
constexpr int row1d_samples(int K, int L) {
  (void)K;
  return L >= 4 ? 32 : 16;
}
constexpr int kRow1dMaxSamples = 32;
constexpr int kRow1dMaxLanes = 512;      // threads per workgroup
constexpr bool row1d_built(int K, int L) { return K >= 3 && row1d_samples(K, L) <= kRow1dMaxSamples; }

// Edge entries a lane publishes of an array of n entries: the first and last R, or all of
// them when there are fewer than 2R.
constexpr int row1d_pub(int n, int R) { return n < 2 * R ? n : 2 * R; }
// Entries of array `a` (0: the samples; 1 + 2(l-1) + s: level l, sub-band s).
constexpr int row1d_len(int S, int a) { return a == 0 ? S : S >> (1 + (a - 1) / 2); }
// Offset of array `a` inside a lane's published edges.
constexpr int row1d_edge_off(int K, int S, int a) {
  int off = 0;
  for (int i = 0; i < a; ++i) off += row1d_pub(row1d_len(S, i), K / 2);
  return off;
}

// Floats of LDS per lane: the lane's S samples (plus a pad that makes the stride an odd
// number of 16-byte units) or its published edges, whichever is larger.
constexpr int row1d_slot(int K, int L) {
  const int S = row1d_samples(K, L);
  const int halo = row1d_edge_off(K, S, 1 + 2 * L);
  int f = S + 4 > halo ? S + 4 : halo;
  f = (f + 3) / 4 * 4;
  if ((f / 4) % 2 == 0) f += 4;
  return f;
}

struct Row1D {
  int C, N;
  int nl;        // lanes that hold samples: ceil(N / S)
  int vec_ok;    // rows are 16-byte sized and aligned
};

// HBM row -> LDS slots (slot of lane j = samples [j*S, (j+1)*S), zeros past N), in two steps
// so that the loads of the next row can be in flight while the current one is computed:
// row1d_fetch issues every 16-byte load of the thread at once (at most S / EV of them, since
// the workgroup has at least as many threads as lanes that hold samples), row1d_commit
// converts and writes them to the slots.  Fast path only: rows are 16-byte sized and aligned,
// so every vector lies wholly inside or wholly outside the row.
template <typename T, int S>
__device__ __forceinline__ void row1d_fetch(const T* __restrict__ row, int N, int tid, int nth,
                                            uint4 (&q)[S / (16 / sizeof(T))]) {
  constexpr int EV = 16 / sizeof(T);
#pragma unroll
  for (int u = 0; u < S / EV; ++u) {
    const int p = (tid + u * nth) * EV;
    q[u].x = 0u; q[u].y = 0u; q[u].z = 0u; q[u].w = 0u;
    if (p < N) q[u] = *reinterpret_cast<const uint4*>(row + p);
  }
}

template <int S, int SLOT, int EV>
__device__ __forceinline__ void row1d_put(float* __restrict__ lds, int p, const float (&vals)[EV]) {
  const int owner = p / S;               // S is a multiple of EV: one owner per vector
  float* dst = lds + owner * SLOT + (p - owner * S);
#pragma unroll
  for (int g = 0; g < EV / 4; ++g) {
    float4 w4;
    w4.x = vals[4 * g]; w4.y = vals[4 * g + 1]; w4.z = vals[4 * g + 2]; w4.w = vals[4 * g + 3];
    reinterpret_cast<float4*>(dst)[g] = w4;
  }
}

template <typename T, int S, int SLOT>
__device__ __forceinline__ void row1d_commit(float* __restrict__ lds, int nl, int tid, int nth,
                                             const uint4 (&q)[S / (16 / sizeof(T))]) {
  constexpr int EV = 16 / sizeof(T);
  const int total = nl * S;
#pragma unroll
  for (int u = 0; u < S / EV; ++u) {
    const int p = (tid + u * nth) * EV;
    if (p < total) {
      float vals[EV];
      if constexpr (sizeof(T) == 4) {
        vals[0] = __uint_as_float(q[u].x); vals[1] = __uint_as_float(q[u].y);
        vals[2] = __uint_as_float(q[u].z); vals[3] = __uint_as_float(q[u].w);
      } else {
        const uint32_t qq[4] = {q[u].x, q[u].y, q[u].z, q[u].w};
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          unpack2<T>(qq[k], vals[2 * k], vals[2 * k + 1]);
        }
      }
      row1d_put<S, SLOT, EV>(lds, p, vals);
    }
  }
}

// Fetch and commit of two rows (x and grad_out) in one call, four vectors of each at a time:
// bounded register use for the kernel that holds many running sums, and the loads of both
// rows share their HBM latency.
template <typename T, int S, int SLOT>
__device__ __forceinline__ void row1d_stage_pair(const T* __restrict__ row0, const T* __restrict__ row1,
                                                 float* __restrict__ lds0, float* __restrict__ lds1, int N, int nl,
                                                 int tid, int nth) {
  constexpr int EV = 16 / sizeof(T);
  constexpr int U = 4;
  const int total = nl * S;
  auto unpack = [](const uint4& q, float (&vals)[EV]) {
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
  };
  for (int v0 = tid; v0 * EV < total; v0 += U * nth) {
    uint4 q0[U], q1[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int p = (v0 + u * nth) * EV;
      q0[u].x = 0u; q0[u].y = 0u; q0[u].z = 0u; q0[u].w = 0u;
      q1[u] = q0[u];
      if (p < N) {
        q0[u] = *reinterpret_cast<const uint4*>(row0 + p);
        q1[u] = *reinterpret_cast<const uint4*>(row1 + p);
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int p = (v0 + u * nth) * EV;
      if (p < total) {
        float vals[EV];
        unpack(q0[u], vals);
        row1d_put<S, SLOT, EV>(lds0, p, vals);
        unpack(q1[u], vals);
        row1d_put<S, SLOT, EV>(lds1, p, vals);
      }
    }
  }
}

// Element-wise staging for rows that are not 16-byte sized or aligned.
template <typename T, int S, int SLOT>
__device__ __forceinline__ void row1d_stage_scalar(const T* __restrict__ row, float* __restrict__ lds, int N,
                                                   int nl, int tid, int nth) {
  constexpr int EV = 16 / sizeof(T);
  const int total = nl * S;
  for (int v = tid; v * EV < total; v += nth) {
    const int p = v * EV;
    float vals[EV];
#pragma unroll
    for (int k = 0; k < EV; ++k) vals[k] = p + k < N ? to_f32<T>(row[p + k]) : 0.f;
    row1d_put<S, SLOT, EV>(lds, p, vals);
  }
}

// LDS slots -> HBM row (entries past N are dropped).
template <typename T, int S, int SLOT>
__device__ __forceinline__ void row1d_unstage(T* __restrict__ row, const float* __restrict__ lds, int N, bool vec,
                                              int tid, int nth) {
  constexpr int EV = 16 / sizeof(T);
  for (int v = tid; v * EV < N; v += nth) {
    const int p = v * EV;
    const int owner = p / S;
    const float* src = lds + owner * SLOT + (p - owner * S);
    float vals[EV];
#pragma unroll
    for (int g = 0; g < EV / 4; ++g) {
      const float4 r4 = reinterpret_cast<const float4*>(src)[g];
      vals[4 * g] = r4.x; vals[4 * g + 1] = r4.y; vals[4 * g + 2] = r4.z; vals[4 * g + 3] = r4.w;
    }
    if (vec && p + EV <= N) {
      uint4 q;
      if constexpr (sizeof(T) == 4) {
        q.x = __float_as_uint(vals[0]); q.y = __float_as_uint(vals[1]);
        q.z = __float_as_uint(vals[2]); q.w = __float_as_uint(vals[3]);
      } else {
        uint32_t qq[4];
#pragma unroll
        for (int k = 0; k < 4; ++k)
          qq[k] = pack2<T>(vals[2 * k], vals[2 * k + 1]);
        q.x = qq[0]; q.y = qq[1]; q.z = qq[2]; q.w = qq[3];
      }
      *reinterpret_cast<uint4*>(row + p) = q;
    } else {
#pragma unroll
      for (int k = 0; k < EV; ++k)
        if (p + k < N) row[p + k] = from_f32<T>(vals[k]);
    }
  }
}

template <int S>
__device__ __forceinline__ void row1d_read_slot(const float* __restrict__ slot, float (&v)[S]) {
#pragma unroll
  for (int g = 0; g < S / 4; ++g) {
    const float4 r4 = reinterpret_cast<const float4*>(slot)[g];
    v[4 * g] = r4.x; v[4 * g + 1] = r4.y; v[4 * g + 2] = r4.z; v[4 * g + 3] = r4.w;
  }
}

template <int S>
__device__ __forceinline__ void row1d_write_slot(float* __restrict__ slot, const float (&v)[S]) {
#pragma unroll
  for (int g = 0; g < S / 4; ++g) {
    float4 w4;
    w4.x = v[4 * g]; w4.y = v[4 * g + 1]; w4.z = v[4 * g + 2]; w4.w = v[4 * g + 3];
    reinterpret_cast<float4*>(slot)[g] = w4;
  }
}

// The lane's pyramid: level l (1-based) has S >> l low-pass and as many high-pass entries.
template <int S, int L>
struct RowPyramid {
  float lo[L][S / 2];
  float hi[L][S / 2];
};

template <int S, int L>
__device__ __forceinline__ void row1d_analysis(const float (&x)[S], RowPyramid<S, L>& py) {
#pragma unroll
  for (int l = 0; l < L; ++l) {
#pragma unroll
    for (int q = 0; q < (S >> (l + 1)); ++q) {
      const float e = l == 0 ? x[2 * q] : py.lo[l > 0 ? l - 1 : 0][2 * q];
      const float o = l == 0 ? x[2 * q + 1] : py.lo[l > 0 ? l - 1 : 0][2 * q + 1];
      py.lo[l][q] = (e + o) * kInvSqrt2;
      py.hi[l][q] = (e - o) * kInvSqrt2;
    }
  }
}

// Publishes the edge entries of array number A (n entries) in the lane's slot.
template <int K, int S, int A, int NA>
__device__ __forceinline__ void row1d_publish(float* __restrict__ slot, const float (&arr)[NA]) {
  constexpr int R = K / 2, n = row1d_len(S, A), OFF = row1d_edge_off(K, S, A);
  static_assert(n <= NA, "array shorter than its level");
  if constexpr (n < 2 * R) {
#pragma unroll
    for (int d = 0; d < n; ++d) slot[OFF + d] = arr[d];
  } else {
#pragma unroll
    for (int d = 0; d < R; ++d) {
      slot[OFF + d] = arr[d];
      slot[OFF + R + d] = arr[n - R + d];
    }
  }
}

template <int K, int S, int L, int l>
__device__ __forceinline__ void row1d_publish_levels(float* __restrict__ slot, const RowPyramid<S, L>& py) {
  if constexpr (l <= L) {
    row1d_publish<K, S, 1 + 2 * (l - 1)>(slot, py.lo[l - 1]);
    row1d_publish<K, S, 2 + 2 * (l - 1)>(slot, py.hi[l - 1]);
    row1d_publish_levels<K, S, L, l + 1>(slot, py);
  }
}

// ext = [R entries to the left | the lane's n entries | R entries to the right] of array A;
// the neighbours' entries come from the slots of the lanes that own them (one or, on coarse
// levels with n < R, several lanes away); beyond either end of the workgroup they are zero.
template <int K, int S, int SLOT, int A, int NA>
__device__ __forceinline__ void row1d_extend(const float* __restrict__ region, int tid, int nth,
                                             const float (&arr)[NA],
                                             float (&ext)[row1d_len(S, A) + 2 * (K / 2)]) {
  constexpr int R = K / 2, n = row1d_len(S, A), OFF = row1d_edge_off(K, S, A);
#pragma unroll
  for (int d = 0; d < R; ++d) {
    {                                              // entry -R + d
      const int e = R - d;                         // distance to the left of entry 0
      const int o = (e + n - 1) / n;               // lanes to the left
      const int loc = o * n - e;                   // its index in that lane's array
      const int pos = n < 2 * R ? loc : R + loc - (n - R);
      ext[d] = tid - o >= 0 ? region[(tid - o) * SLOT + OFF + pos] : 0.f;
    }
    {                                              // entry n + d
      const int o = (n + d) / n;
      const int loc = (n + d) - o * n;
      ext[R + n + d] = tid + o < nth ? region[(tid + o) * SLOT + OFF + loc] : 0.f;
    }
  }
#pragma unroll
  for (int q = 0; q < n; ++q) ext[R + q] = arr[q];
}

template <int K, int n>
__device__ __forceinline__ void row1d_conv(const float (&ext)[n + K - 1], wt_uniform_ptr w, float (&y)[n]) {
#pragma unroll
  for (int k = 0; k < K; ++k) {
    const float wv = w[k];
#pragma unroll
    for (int q = 0; q < n; ++q) y[q] = fmaf(wv, ext[q + k], y[q]);
  }
}

// Synthesis from level l (1-based) down to level 1: `zc` holds Z_{l+1} (n_l entries) on
// entry when l < L; the level-1 reconstruction is added into `out`.
template <int K, int S, int SLOT, int L, int l>
__device__ __forceinline__ void row1d_synth(const RowPyramid<S, L>& py, const float* __restrict__ region, int tid,
                                            int nth, wt_uniform_ptr fwc, float (&zc)[S / 2], float (&out)[S]) {
  if constexpr (l >= 1) {
    constexpr int R = K / 2;
    constexpr int n = S >> l;
    float ylo[n], yhi[n];
#pragma unroll
    for (int q = 0; q < n; ++q) { ylo[q] = l < L ? zc[q] : 0.f; yhi[q] = 0.f; }
    {
      float ext[n + 2 * R];
      row1d_extend<K, S, SLOT, 1 + 2 * (l - 1)>(region, tid, nth, py.lo[l - 1], ext);
      row1d_conv<K, n>(ext, fwc + (1 + 2 * (l - 1)) * K, ylo);
    }
    {
      float ext[n + 2 * R];
      row1d_extend<K, S, SLOT, 2 + 2 * (l - 1)>(region, tid, nth, py.hi[l - 1], ext);
      row1d_conv<K, n>(ext, fwc + (2 + 2 * (l - 1)) * K, yhi);
    }
    if constexpr (l > 1) {
#pragma unroll
      for (int q = 0; q < n; ++q) {
        zc[2 * q] = (ylo[q] + yhi[q]) * kInvSqrt2;       // ylo[q] was read from zc[q] before: q <= 2q
        zc[2 * q + 1] = (ylo[q] - yhi[q]) * kInvSqrt2;
      }
    } else {
#pragma unroll
      for (int q = 0; q < n; ++q) {
        out[2 * q] += (ylo[q] + yhi[q]) * kInvSqrt2;
        out[2 * q + 1] += (ylo[q] - yhi[q]) * kInvSqrt2;
      }
    }
    row1d_synth<K, S, SLOT, L, l - 1>(py, region, tid, nth, fwc, zc, out);
  }
}

// Forward / input-gradient kernel.  Persistent: grid = min(rows, resident workgroups), block =
// lanes (multiple of 64, >= ceil(N / S)), dynamic LDS = 2 * block * SLOT floats: two slot
// regions that alternate between rows.  The next row of the workgroup is fetched into
// registers while the current one is computed and committed to the other region before the
// current outputs are stored, so that loads never wait behind stores; three barriers per row.
template <typename T, int K, int L>
__global__ __launch_bounds__(kRow1dMaxLanes) void wt1d_row_kernel(const T* __restrict__ x, T* __restrict__ out,
                                                                   const float* __restrict__ fw,
                                                                   const float* __restrict__ fb, Row1D pl,
                                                                   int nrows) {
  WT_SHARED_FLOATS(lds);
  constexpr int R = K / 2;
  constexpr int S = row1d_samples(K, L);
  constexpr int SLOT = row1d_slot(K, L);
  constexpr int NF = 1 + 2 * L;
  constexpr int EV = 16 / sizeof(T);
  const int tid = threadIdx.x, nth = blockDim.x;
  const bool fast = pl.vec_ok != 0 && pl.N % EV == 0;
  float* cur = lds;
  float* nxt = lds + nth * SLOT;

  uint4 q[S / EV];
  if (static_cast<int>(blockIdx.x) < nrows) {
    const T* xrow = x + static_cast<size_t>(blockIdx.x) * pl.N;
    if (fast) {
      row1d_fetch<T, S>(xrow, pl.N, tid, nth, q);
      row1d_commit<T, S, SLOT>(cur, pl.nl, tid, nth, q);
    } else {
      row1d_stage_scalar<T, S, SLOT>(xrow, cur, pl.N, pl.nl, tid, nth);
    }
  }
  WT_LDS_BARRIER();
  for (int rv = blockIdx.x; rv < nrows; rv += gridDim.x) {
    const int row = WT_UNIFORM(rv);
    const int c = row % pl.C;
    const bool more = row + static_cast<int>(gridDim.x) < nrows;
    const T* xnext = x + static_cast<size_t>(more ? row + gridDim.x : row) * pl.N;
    wt_uniform_ptr fwc = (wt_uniform_ptr)(fw + static_cast<size_t>(c) * NF * K);
    float* slot = cur + tid * SLOT;
    float xs[S];
    if (tid < pl.nl) {
      row1d_read_slot<S>(slot, xs);
    } else {
#pragma unroll
      for (int e = 0; e < S; ++e) xs[e] = 0.f;
    }
    if (fast && more) row1d_fetch<T, S>(xnext, pl.N, tid, nth, q);
    RowPyramid<S, L> py;
    row1d_analysis<S, L>(xs, py);
    // the slot held this lane's samples only: it can take the lane's edges right away
    row1d_publish<K, S, 0>(slot, xs);
    row1d_publish_levels<K, S, L, 1>(slot, py);
    WT_LDS_BARRIER();

    float o[S];
    {
      const float bias = fb[c];
#pragma unroll
      for (int e = 0; e < S; ++e) o[e] = bias;
      float ext[S + 2 * R];
      row1d_extend<K, S, SLOT, 0>(cur, tid, nth, xs, ext);
      row1d_conv<K, S>(ext, fwc, o);
    }
    float zc[S / 2];
#pragma unroll
    for (int e = 0; e < S / 2; ++e) zc[e] = 0.f;
    row1d_synth<K, S, SLOT, L, L>(py, cur, tid, nth, fwc, zc, o);
    WT_LDS_BARRIER();            // every neighbour has read this lane's edges
    row1d_write_slot<S>(slot, o);
    if (more) {                  // the other region is idle: nothing has read it since the last barrier but one
      if (fast)
        row1d_commit<T, S, SLOT>(nxt, pl.nl, tid, nth, q);
      else
        row1d_stage_scalar<T, S, SLOT>(xnext, nxt, pl.N, pl.nl, tid, nth);
    }
    WT_LDS_BARRIER();
    row1d_unstage<T, S, SLOT>(out + static_cast<size_t>(row) * pl.N, cur, pl.N, pl.vec_ok != 0, tid, nth);
    float* t = cur; cur = nxt; nxt = t;
  }
}

// sum_q g[q] * ext[q + k] for the K taps of one filter
template <int K, int n, int NG>
__device__ __forceinline__ void row1d_corr(const float (&ext)[n + K - 1], const float (&g)[NG], float (&acc)[K]) {
#pragma unroll
  for (int q = 0; q < n; ++q)
#pragma unroll
    for (int k = 0; k < K; ++k) acc[k] = fmaf(g[q], ext[q + k], acc[k]);
}

// Levels l..L of the parameter-gradient sums; `gprev` = low-pass of grad_out at level l-1
// (2n entries), analysed one level at a time so that only one level of it is live.
template <int K, int S, int SLOT, int L, int l>
__device__ __forceinline__ void row1d_wgrad_levels(const RowPyramid<S, L>& py, const float* __restrict__ region,
                                                   int tid, int nth, const float (&gprev)[(S >> (l - 1))],
                                                   float (&acc)[1 + 2 * L][K]) {
  constexpr int R = K / 2;
  constexpr int n = S >> l;
  float glo[n], ghi[n];
#pragma unroll
  for (int q = 0; q < n; ++q) {
    glo[q] = (gprev[2 * q] + gprev[2 * q + 1]) * kInvSqrt2;
    ghi[q] = (gprev[2 * q] - gprev[2 * q + 1]) * kInvSqrt2;
  }
  {
    float ext[n + 2 * R];
    row1d_extend<K, S, SLOT, 1 + 2 * (l - 1)>(region, tid, nth, py.lo[l - 1], ext);
    row1d_corr<K, n>(ext, glo, acc[1 + 2 * (l - 1)]);
  }
  {
    float ext[n + 2 * R];
    row1d_extend<K, S, SLOT, 2 + 2 * (l - 1)>(region, tid, nth, py.hi[l - 1], ext);
    row1d_corr<K, n>(ext, ghi, acc[2 + 2 * (l - 1)]);
  }
  if constexpr (l < L) row1d_wgrad_levels<K, S, SLOT, L, l + 1>(py, region, tid, nth, glo, acc);
}

// Parameter gradients, first stage.  grid = (C, nchunk), block = lanes, dynamic LDS =
// 2 * block * SLOT floats (x slots, then grad_out slots).  A workgroup walks `per_chunk` rows
// of one channel; every lane keeps K sums per filter in registers.  Output layout as the
// tiled kernel: partial[chunk][c][(1 + 2L) * K + 1].
template <typename T, int K, int L>
__global__ __launch_bounds__(kRow1dMaxLanes) void wt1d_row_wgrad_kernel(const T* __restrict__ x,
                                                                         const T* __restrict__ g,
                                                                         float* __restrict__ partial, Row1D pl,
                                                                         int B, int per_chunk) {
  WT_SHARED_FLOATS(lds);
  constexpr int R = K / 2;
  constexpr int S = row1d_samples(K, L);
  constexpr int SLOT = row1d_slot(K, L);
  constexpr int NF = 1 + 2 * L;
  const int c = blockIdx.x;
  const int chunk = blockIdx.y;
  const int tid = threadIdx.x, nth = blockDim.x;
  float* xlds = lds;
  float* glds = lds + nth * SLOT;
  float* slot = xlds + tid * SLOT;
  const float* gslot = glds + tid * SLOT;

  constexpr int EV = 16 / sizeof(T);
  const bool fast = pl.vec_ok != 0 && pl.N % EV == 0;

  float acc[NF][K];
  float gsum = 0.f;
#pragma unroll
  for (int f = 0; f < NF; ++f)
#pragma unroll
    for (int k = 0; k < K; ++k) acc[f][k] = 0.f;

  const int b_end = (chunk + 1) * per_chunk < B ? (chunk + 1) * per_chunk : B;
  for (int b = chunk * per_chunk; b < b_end; ++b) {
    const size_t roff = (static_cast<size_t>(b) * pl.C + c) * pl.N;
    if (fast) {
      row1d_stage_pair<T, S, SLOT>(x + roff, g + roff, xlds, glds, pl.N, pl.nl, tid, nth);
    } else {
      row1d_stage_scalar<T, S, SLOT>(x + roff, xlds, pl.N, pl.nl, tid, nth);
      row1d_stage_scalar<T, S, SLOT>(g + roff, glds, pl.N, pl.nl, tid, nth);
    }
    WT_LDS_BARRIER();
    float xs[S], gs[S];
    if (tid < pl.nl) {
      row1d_read_slot<S>(slot, xs);
      row1d_read_slot<S>(gslot, gs);
    } else {
#pragma unroll
      for (int q = 0; q < S; ++q) { xs[q] = 0.f; gs[q] = 0.f; }
    }
    RowPyramid<S, L> py;
    row1d_analysis<S, L>(xs, py);
    row1d_publish<K, S, 0>(slot, xs);
    row1d_publish_levels<K, S, L, 1>(slot, py);
    WT_LDS_BARRIER();
    {
      float ext[S + 2 * R];
      row1d_extend<K, S, SLOT, 0>(xlds, tid, nth, xs, ext);
      row1d_corr<K, S>(ext, gs, acc[0]);
#pragma unroll
      for (int q = 0; q < S; ++q) gsum += gs[q];
    }
    row1d_wgrad_levels<K, S, SLOT, L, 1>(py, xlds, tid, nth, gs, acc);
    WT_LDS_BARRIER();            // the next row's staging overwrites the edges read above
  }

  constexpr int NRED = NF * K + 1;
  float* red = lds;              // [waves][NRED]
  const int wave = tid >> 6, lane = tid & (kWave - 1);
#pragma unroll
  for (int f = 0; f < NF; ++f)
#pragma unroll
    for (int k = 0; k < K; ++k) {
      const float v = wave_sum(acc[f][k]);
      if (lane == 0) red[wave * NRED + f * K + k] = v;
    }
  {
    const float v = wave_sum(gsum);
    if (lane == 0) red[wave * NRED + NRED - 1] = v;
  }
  WT_LDS_BARRIER();
  float* dst = partial + (static_cast<size_t>(chunk) * pl.C + c) * NRED;
  const int nwaves = nth >> 6;
  for (int o = tid; o < NRED; o += nth) {
    float v = 0.f;
    for (int wv = 0; wv < nwaves; ++wv) v += red[wv * NRED + o];
    dst[o] = v;
  }
}

}  // namespace wt
