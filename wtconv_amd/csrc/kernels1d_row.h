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
//
// A workgroup works on rows of ONE channel (grid = channels x batch chunks), and folds that
// channel's parameters itself when it starts (gamma * w, taps reversed for the input gradient):
// one entry per lane, read back as wave-uniform values -- no fold launch, no folded table in
// HBM.  The backward pass is one kernel: the row of x and the row of grad_out are read once and
// give grad_x and the running sums of the parameter gradients; the workgroup that finishes a
// channel last (a ticket per channel) sums the chunks' partial sums in chunk order and writes
// the channel's parameter gradients.
#pragma once

#include "common.h"
#include "kernels1d.h"
#include "wgrad_finish.h"

namespace wt {

// Samples per lane S: a multiple of 2^L (the pyramid of a lane is local) and of 8 (16-byte vectors of either
// dtype): 16 or 32.  16 wherever the row fits the workgroup with it (twice the lanes per row, half the registers
// per lane: more waves in flight, which is what these latency-bound kernels need), 32 for longer rows and for
// five levels.
constexpr int kRow1dMaxSamples = 32;
constexpr int kRow1dMaxLanes = 512;      // threads per workgroup
constexpr bool row1d_built(int K, int L, int S) {
  return K >= 3 && (S == 16 || S == 32) && S % (1 << L) == 0;
}

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
constexpr int row1d_slot(int K, int L, int S) {
  const int halo = row1d_edge_off(K, S, 1 + 2 * L);
  int f = S + 4 > halo ? S + 4 : halo;
  f = (f + 3) / 4 * 4;
  if ((f / 4) % 2 == 0) f += 4;
  return f;
}

// Zero slots on either side of a region's `block` lane slots: a lane reads the edges of up to ceil(R / n) lanes
// away (n = entries per lane at the coarsest level), and beyond either end of the row those reads land here --
// no condition, no branch around the read, every edge at a constant offset from the lane's own slot.
constexpr int row1d_guard(int K, int L, int S) {
  const int nmin = S >> L;
  const int R = K / 2;
  return nmin < 1 ? R : (R + nmin - 1) / nmin;
}
// Floats of one region (guards included) for a workgroup of `block` lanes.
constexpr size_t row1d_region(int K, int L, int S, int block) {
  return static_cast<size_t>(block + 2 * row1d_guard(K, L, S)) * row1d_slot(K, L, S);
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
// STREAM: the loads are marked non-temporal (measured: pays in the whole-backward kernel, which reads two rows per
// row it writes, not in the forward kernel).
template <typename T, int S, bool STREAM = false>
__device__ __forceinline__ void row1d_fetch(const T* __restrict__ row, int N, int tid, int nth,
                                            uint4 (&q)[S / (16 / sizeof(T))]) {
  constexpr int EV = 16 / sizeof(T);
#pragma unroll
  for (int u = 0; u < S / EV; ++u) {
    const int p = (tid + u * nth) * EV;
    q[u].x = 0u; q[u].y = 0u; q[u].z = 0u; q[u].w = 0u;
    if (p < N) {
      if constexpr (STREAM) q[u] = load_stream_u4(row + p);
      else q[u] = *reinterpret_cast<const uint4*>(row + p);
    }
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
      store_stream_u4(row + p, q);       // written once, read by another kernel: non-temporal
    } else {
#pragma unroll
      for (int k = 0; k < EV; ++k)
        if (p + k < N) row[p + k] = from_f32<T>(vals[k]);
    }
  }
}

// Zeroes the guard slots of the `nregion` regions that start at `lds` (once per workgroup: nothing else writes them).
template <int K, int L, int S>
__device__ __forceinline__ void row1d_zero_guards(float* __restrict__ lds, int nregion, int tid, int nth) {
  constexpr int SLOT = row1d_slot(K, L, S), G = row1d_guard(K, L, S);
  const int rfl = (nth + 2 * G) * SLOT;
  for (int r = 0; r < nregion; ++r)
    for (int i = tid; i < 2 * G * SLOT; i += nth) {
      const int off = i < G * SLOT ? i : rfl - 2 * G * SLOT + i;
      lds[r * rfl + off] = 0.f;
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

// Scaling.  The butterflies here are sums and differences without their 1/sqrt(2): level l's coefficients are
// 2^(l/2) times the orthonormal ones of wtconv/util/wavelet.py:46-59.  The folded weights of level l carry 2^-l
// (row1d_fold), which makes every level's reconstruction come out exactly scaled -- each inverse butterfly and each
// repeat of a coarse value owes 2^(-1/2), l of them in all -- and the correlation sums of level l (two pyramids, each
// 2^(l/2) up) are brought back by 2^-l when they leave the registers (row1d_store_partial).  Only powers of two are
// moved, which is exact; the 2 n multiplications per level and pass, and their roundings, are gone.
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
      py.lo[l][q] = e + o;
      py.hi[l][q] = e - o;
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
// levels with n < R, several lanes away); beyond either end of the workgroup those are the
// region's zero guard slots.
template <int K, int S, int SLOT, int A, int NA>
__device__ __forceinline__ void row1d_extend(const float* __restrict__ region, int tid, int nth,
                                             const float (&arr)[NA],
                                             float (&ext)[row1d_len(S, A) + 2 * (K / 2)]) {
  (void)nth;
  constexpr int R = K / 2, n = row1d_len(S, A), OFF = row1d_edge_off(K, S, A);
  const float* own = region + tid * SLOT;
#pragma unroll
  for (int d = 0; d < R; ++d) {
    {                                              // entry -R + d
      const int e = R - d;                         // distance to the left of entry 0
      const int o = (e + n - 1) / n;               // lanes to the left
      const int loc = o * n - e;                   // its index in that lane's array
      const int pos = n < 2 * R ? loc : R + loc - (n - R);
      ext[d] = own[-o * SLOT + OFF + pos];
    }
    {                                              // entry n + d
      const int o = (n + d) / n;
      const int loc = (n + d) - o * n;
      ext[R + n + d] = own[o * SLOT + OFF + loc];
    }
  }
#pragma unroll
  for (int q = 0; q < n; ++q) ext[R + q] = arr[q];
}

// The edges of every array of a lane's neighbours, fetched in one go (all the LDS reads of a row are in flight together
// and waited for once): v[A][0..R) the R entries to the left of the lane's array A, v[A][R..2R) the R to its right.
template <int K, int L>
struct RowEdges { float v[1 + 2 * L][2 * (K / 2) > 0 ? 2 * (K / 2) : 1]; };

template <int K, int S, int SLOT, int L, int A>
__device__ __forceinline__ void row1d_load_edges_from(const float* __restrict__ own, RowEdges<K, L>& ed) {
  if constexpr (A <= 2 * L) {
    constexpr int R = K / 2, n = row1d_len(S, A), OFF = row1d_edge_off(K, S, A);
#pragma unroll
    for (int d = 0; d < R; ++d) {
      {
        const int e = R - d, o = (e + n - 1) / n, loc = o * n - e;
        const int pos = n < 2 * R ? loc : R + loc - (n - R);
        ed.v[A][d] = own[-o * SLOT + OFF + pos];
      }
      {
        const int o = (n + d) / n, loc = (n + d) - o * n;
        ed.v[A][R + d] = own[o * SLOT + OFF + loc];
      }
    }
    row1d_load_edges_from<K, S, SLOT, L, A + 1>(own, ed);
  }
}

template <int K, int S, int SLOT, int L>
__device__ __forceinline__ void row1d_load_edges(const float* __restrict__ region, int tid, RowEdges<K, L>& ed) {
  row1d_load_edges_from<K, S, SLOT, L, 0>(region + tid * SLOT, ed);
}

// ext of array A from edges fetched earlier
template <int K, int S, int L, int A, int NA>
__device__ __forceinline__ void row1d_extend_with(const RowEdges<K, L>& ed, const float (&arr)[NA],
                                                  float (&ext)[row1d_len(S, A) + 2 * (K / 2)]) {
  constexpr int R = K / 2, n = row1d_len(S, A);
#pragma unroll
  for (int d = 0; d < R; ++d) { ext[d] = ed.v[A][d]; ext[R + n + d] = ed.v[A][R + d]; }
#pragma unroll
  for (int q = 0; q < n; ++q) ext[R + q] = arr[q];
}

// Folded parameters of one channel: entry f * K + k = gamma[f] * w[f][k] (k reversed when flip != 0), f = 0 base
// conv, f = 1 + 2 (l - 1) + s level l sub-band s.  The same products as fold_params_kernel forms.
template <int K, int L>
using RowWeights = LaneTable<(1 + 2 * L) * K>;

template <int K, int L>
__device__ __forceinline__ void row1d_fold(const ParamTable& p, int pdtype, int c, int flip, RowWeights<K, L>& tab) {
  tab.fill([&](int i) {
    const int f = i / K, t = i - f * K;
    const int ts = flip ? K - 1 - t : t;
    float v = 0.f;
    if (f == 0) v = load_param(p.base_weight, pdtype, c * K + ts) * load_param(p.base_scale, pdtype, c);
#pragma unroll
    for (int l = 0; l < L; ++l) {
      if (f >= 1 + 2 * l && f < 3 + 2 * l) {
        const int ch = c * 2 + (f - 1 - 2 * l);
        v = load_param(p.wt_weight[l], pdtype, ch * K + ts) * load_param(p.wt_scale[l], pdtype, ch) *
            (1.f / static_cast<float>(2 << l));          // 2^-(level): see "Scaling"
      }
    }
    return v;
  });
}

// y += (filter F of the channel) (*) ext
template <int K, int L, int F, int n>
__device__ __forceinline__ void row1d_conv(const float (&ext)[n + K - 1], const RowWeights<K, L>& w, float (&y)[n]) {
#pragma unroll
  for (int k = 0; k < K; ++k) {
    const float wv = w.get(F * K + k);
#pragma unroll
    for (int q = 0; q < n; ++q) y[q] = fmaf(wv, ext[q + k], y[q]);
  }
}

// Synthesis from level l (1-based) down to level 1: `zc` holds Z_{l+1} (n_l entries) on
// entry when l < L; the level-1 reconstruction is added into `out`.
template <int K, int S, int SLOT, int L, int l>
__device__ __forceinline__ void row1d_synth(const RowPyramid<S, L>& py, const float* __restrict__ region, int tid,
                                            int nth, const RowWeights<K, L>& fwc, float (&zc)[S / 2], float (&out)[S]) {
  if constexpr (l >= 1) {
    constexpr int R = K / 2;
    constexpr int n = S >> l;
    float ylo[n], yhi[n];
#pragma unroll
    for (int q = 0; q < n; ++q) { ylo[q] = l < L ? zc[q] : 0.f; yhi[q] = 0.f; }
    {
      float ext[n + 2 * R];
      row1d_extend<K, S, SLOT, 1 + 2 * (l - 1)>(region, tid, nth, py.lo[l - 1], ext);
      row1d_conv<K, L, 1 + 2 * (l - 1), n>(ext, fwc, ylo);
    }
    {
      float ext[n + 2 * R];
      row1d_extend<K, S, SLOT, 2 + 2 * (l - 1)>(region, tid, nth, py.hi[l - 1], ext);
      row1d_conv<K, L, 2 + 2 * (l - 1), n>(ext, fwc, yhi);
    }
    if constexpr (l > 1) {
#pragma unroll
      for (int q = 0; q < n; ++q) {
        zc[2 * q] = ylo[q] + yhi[q];       // ylo[q] was read from zc[q] before: q <= 2q
        zc[2 * q + 1] = ylo[q] - yhi[q];
      }
    } else {
#pragma unroll
      for (int q = 0; q < n; ++q) {
        out[2 * q] += ylo[q] + yhi[q];
        out[2 * q + 1] += ylo[q] - yhi[q];
      }
    }
    row1d_synth<K, S, SLOT, L, l - 1>(py, region, tid, nth, fwc, zc, out);
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
    glo[q] = gprev[2 * q] + gprev[2 * q + 1];
    ghi[q] = gprev[2 * q] - gprev[2 * q + 1];
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

// The per-chunk record of a workgroup's running sums: cross-lane sums, then cross-wave through `red`
// ([waves][NRED] floats of LDS, idle by now), into partial[chunk][c][NF * K + 1].
template <int K, int NF, bool SHARED = false>
__device__ __forceinline__ void row1d_store_partial(const float (&acc)[NF][K], float gsum, float* __restrict__ red,
                                                    float* __restrict__ dst, int tid, int nth) {
  constexpr int NRED = NF * K + 1;
  const int wave = tid >> 6, lane = tid & (kWave - 1);
#pragma unroll
  for (int f = 0; f < NF; ++f)
#pragma unroll
    for (int k = 0; k < K; ++k) {
      // the sums of level l were formed from coefficients 2^(l/2) times the orthonormal ones on either side
      const float v = wave_sum(acc[f][k]) * (f == 0 ? 1.f : 1.f / static_cast<float>(2 << ((f - 1) / 2)));
      if (lane == 0) red[wave * NRED + f * K + k] = v;
    }
  {
    const float v = wave_sum(gsum);
    if (lane == 0) red[wave * NRED + NRED - 1] = v;
  }
  WT_LDS_BARRIER();
  const int nwaves = nth >> 6;
  for (int o = tid; o < NRED; o += nth) {
    float v = 0.f;
    for (int wv = 0; wv < nwaves; ++wv) v += red[wv * NRED + o];
    if constexpr (SHARED) store_shared_f32(dst + o, v);
    else dst[o] = v;
  }
}

// Fused backward kernel, before the barrier: level l of a lane's pyramid from level l - 1 (`prev`), its edges
// published at once; only the low-pass of the current level stays live (the levels are formed again, one at a time,
// after the barrier: two operations per coefficient, against sixty registers for a whole pyramid).
template <int K, int S, int L, int l>
__device__ __forceinline__ void row1d_publish_chain(float* __restrict__ slot, const float (&prev)[(S >> (l - 1))]) {
  constexpr int n = S >> l;
  float lo[n], hi[n];
#pragma unroll
  for (int q = 0; q < n; ++q) {
    lo[q] = prev[2 * q] + prev[2 * q + 1];
    hi[q] = prev[2 * q] - prev[2 * q + 1];
  }
  row1d_publish<K, S, 1 + 2 * (l - 1)>(slot, lo);
  row1d_publish<K, S, 2 + 2 * (l - 1)>(slot, hi);
  if constexpr (l < L) row1d_publish_chain<K, S, L, l + 1>(slot, lo);
}

// Fused backward kernel, after the barrier: levels l..L of both halves of the backward pass, walking from the
// finest level down.  `xprev` / `gprev` = low-pass of x / grad_out at level l - 1.  Per level: the four coefficient
// arrays; the correlation sums of x's with grad_out's; the level's contribution to grad_x.  That contribution is
// added to the samples directly: the inverse transform is linear, and a reconstruction with zero detail below level
// l is the level-l result repeated 2^(l-1) times and scaled by 2^(-(l-1)/2), so the levels need not be visited
// coarsest first and no level's coefficients outlive its visit.
template <int K, int S, int SLOT, int L, int l>
__device__ __forceinline__ void row1d_bwd_levels(const float* __restrict__ xregion, const float* __restrict__ gregion,
                                                 int tid, int nth, const RowWeights<K, L>& fwc,
                                                 const float (&xprev)[(S >> (l - 1))],
                                                 const float (&gprev)[(S >> (l - 1))], float (&acc)[1 + 2 * L][K],
                                                 float (&o)[S]) {
  constexpr int R = K / 2;
  constexpr int n = S >> l;
  constexpr int A = 1 + 2 * (l - 1);
  float xlo[n], glo[n], ylo[n], yhi[n];
#pragma unroll
  for (int q = 0; q < n; ++q) { ylo[q] = 0.f; yhi[q] = 0.f; }
  {
    float xhi[n], ghi[n];
#pragma unroll
    for (int q = 0; q < n; ++q) {
      xlo[q] = xprev[2 * q] + xprev[2 * q + 1];
      xhi[q] = xprev[2 * q] - xprev[2 * q + 1];
      glo[q] = gprev[2 * q] + gprev[2 * q + 1];
      ghi[q] = gprev[2 * q] - gprev[2 * q + 1];
    }
    {
      float ext[n + 2 * R];
      row1d_extend<K, S, SLOT, A + 1>(xregion, tid, nth, xhi, ext);
      row1d_corr<K, n>(ext, ghi, acc[A + 1]);
    }
    {
      float ext[n + 2 * R];
      row1d_extend<K, S, SLOT, A + 1>(gregion, tid, nth, ghi, ext);
      row1d_conv<K, L, A + 1, n>(ext, fwc, yhi);
    }
    pin_values(yhi);
    WT_CHUNK_FENCE();      // (the edge reads of the next part stay below: one part's edges live at a time)
  }
  {
    float ext[n + 2 * R];
    row1d_extend<K, S, SLOT, A>(xregion, tid, nth, xlo, ext);
    row1d_corr<K, n>(ext, glo, acc[A]);
  }
  {
    float ext[n + 2 * R];
    row1d_extend<K, S, SLOT, A>(gregion, tid, nth, glo, ext);
    row1d_conv<K, L, A, n>(ext, fwc, ylo);
  }
  // (one inverse butterfly and l - 1 repeats: no factor left, see "Scaling" above)
  constexpr int REP = 1 << (l - 1);
#pragma unroll
  for (int q = 0; q < n; ++q) {
    const float ev = ylo[q] + yhi[q], od = ylo[q] - yhi[q];
#pragma unroll
    for (int r = 0; r < REP; ++r) {
      o[(2 * q) * REP + r] += ev;
      o[(2 * q + 1) * REP + r] += od;
    }
  }
  pin_values(o);
  WT_CHUNK_FENCE();
  if constexpr (l < L) row1d_bwd_levels<K, S, SLOT, L, l + 1>(xregion, gregion, tid, nth, fwc, xlo, glo, acc, o);
}

// The forward / input-gradient kernel's walk over the levels, finest first, on the same terms: per level the two
// coefficient arrays, their convolutions, and the level's contribution added to the samples directly.
template <int K, int S, int SLOT, int L, int l>
__device__ __forceinline__ void row1d_fwd_levels(const RowEdges<K, L>& ed, const RowWeights<K, L>& fwc,
                                                 const float (&xprev)[(S >> (l - 1))], float (&o)[S]) {
  constexpr int R = K / 2;
  constexpr int n = S >> l;
  constexpr int A = 1 + 2 * (l - 1);
  float xlo[n], ylo[n], yhi[n];
#pragma unroll
  for (int q = 0; q < n; ++q) { ylo[q] = 0.f; yhi[q] = 0.f; }
  {
    float xhi[n];
#pragma unroll
    for (int q = 0; q < n; ++q) {
      xlo[q] = xprev[2 * q] + xprev[2 * q + 1];
      xhi[q] = xprev[2 * q] - xprev[2 * q + 1];
    }
    float ext[n + 2 * R];
    row1d_extend_with<K, S, L, A + 1>(ed, xhi, ext);
    row1d_conv<K, L, A + 1, n>(ext, fwc, yhi);
  }
  {
    float ext[n + 2 * R];
    row1d_extend_with<K, S, L, A>(ed, xlo, ext);
    row1d_conv<K, L, A, n>(ext, fwc, ylo);
  }
  constexpr int REP = 1 << (l - 1);
#pragma unroll
  for (int q = 0; q < n; ++q) {
    const float ev = ylo[q] + yhi[q], od = ylo[q] - yhi[q];
#pragma unroll
    for (int r = 0; r < REP; ++r) {
      o[(2 * q) * REP + r] += ev;
      o[(2 * q + 1) * REP + r] += od;
    }
  }
  if constexpr (l < L) row1d_fwd_levels<K, S, SLOT, L, l + 1>(ed, fwc, xlo, o);
}

// Forward / input-gradient kernel.  grid = (channels, batch chunks), block = lanes (multiple of 64,
// >= ceil(N / S)), dynamic LDS = one slot region (row1d_region floats).  A workgroup walks the rows (b, c) of
// its chunk of batch items; the next row is fetched into registers while the current one is computed and
// committed to the slots once the current outputs have left them.  One region instead of two alternating
// ones: half the LDS per workgroup, i.e. twice the workgroups per CU, which pays more here than the two
// barriers per row it costs.  flip != 0: the input gradient (taps reversed, no bias).
template <typename T, int K, int L, int S>
__global__ __launch_bounds__(kRow1dMaxLanes) void wt1d_row_kernel(const T* __restrict__ x, T* __restrict__ out,
                                                                   const ParamTable prm, int pdtype, int flip,
                                                                   Row1D pl, int B, int per_chunk) {
  WT_SHARED_FLOATS(lds);
  constexpr int R = K / 2;
  constexpr int SLOT = row1d_slot(K, L, S);
  constexpr int EV = 16 / sizeof(T);
  const int tid = threadIdx.x, nth = blockDim.x;
  const int c = blockIdx.x;
  const int b_begin = static_cast<int>(blockIdx.y) * per_chunk;
  const int b_end = b_begin + per_chunk < B ? b_begin + per_chunk : B;
  const bool fast = pl.vec_ok != 0 && pl.N % EV == 0;
  constexpr int G = row1d_guard(K, L, S);
  float* cur = lds + G * SLOT;                      // (the region points at the slot of lane 0, behind its left guard)
  row1d_zero_guards<K, L, S>(lds, 1, tid, nth);
  auto row_of = [&](int b) { return (static_cast<size_t>(b) * pl.C + c) * pl.N; };

  uint4 q[S / EV];
  if (b_begin < b_end && fast) row1d_fetch<T, S>(x + row_of(b_begin), pl.N, tid, nth, q);
  RowWeights<K, L> fwc;                 // (its parameter loads share the latency of the first row's)
  row1d_fold<K, L>(prm, pdtype, c, flip, fwc);
  const float bias = (!flip && prm.base_bias != nullptr)
                         ? load_param(prm.base_bias, pdtype, c) * load_param(prm.base_scale, pdtype, c) : 0.f;
  if (b_begin < b_end) {
    if (fast)
      row1d_commit<T, S, SLOT>(cur, pl.nl, tid, nth, q);
    else
      row1d_stage_scalar<T, S, SLOT>(x + row_of(b_begin), cur, pl.N, pl.nl, tid, nth);
  }
  WT_LDS_BARRIER();
  for (int bv = b_begin; bv < b_end; ++bv) {
    const int b = WT_UNIFORM(bv);
    const bool more = b + 1 < b_end;
    const T* xnext = x + row_of(more ? b + 1 : b);
    float* slot = cur + tid * SLOT;
    float xs[S];
    if (tid < pl.nl) {
      row1d_read_slot<S>(slot, xs);
    } else {
#pragma unroll
      for (int e = 0; e < S; ++e) xs[e] = 0.f;
    }
    if (fast && more) row1d_fetch<T, S>(xnext, pl.N, tid, nth, q);
    // the slot held this lane's samples only: it can take the lane's edges right away
    row1d_publish<K, S, 0>(slot, xs);
    row1d_publish_chain<K, S, L, 1>(slot, xs);
    WT_LDS_BARRIER();
    pin_values(xs);              // (the levels are formed again below, one at a time, not kept across the barrier)

    RowEdges<K, L> ed;
    row1d_load_edges<K, S, SLOT, L>(cur, tid, ed);
    float o[S];
    {
#pragma unroll
      for (int e = 0; e < S; ++e) o[e] = bias;
      float ext[S + 2 * R];
      row1d_extend_with<K, S, L, 0>(ed, xs, ext);
      row1d_conv<K, L, 0, S>(ext, fwc, o);
    }
    row1d_fwd_levels<K, S, SLOT, L, 1>(ed, fwc, xs, o);
    WT_LDS_BARRIER();            // every neighbour has read this lane's edges
    row1d_write_slot<S>(slot, o);
    WT_LDS_BARRIER();
    row1d_unstage<T, S, SLOT>(out + row_of(b), cur, pl.N, pl.vec_ok != 0, tid, nth);
    WT_LDS_BARRIER();            // the outputs have left the slots
    if (more) {
      if (fast)
        row1d_commit<T, S, SLOT>(cur, pl.nl, tid, nth, q);
      else
        row1d_stage_scalar<T, S, SLOT>(xnext, cur, pl.N, pl.nl, tid, nth);
    }
    WT_LDS_BARRIER();
  }
}

// Parameter gradients, first stage.  grid = (C, nchunk), block = lanes, dynamic LDS =
// 2 * block * SLOT floats (x slots, then grad_out slots).  A workgroup walks `per_chunk` rows
// of one channel; every lane keeps K sums per filter in registers.  Output layout as the
// tiled kernel: partial[chunk][c][(1 + 2L) * K + 1].
template <typename T, int K, int L, int S>
__global__ __launch_bounds__(kRow1dMaxLanes) void wt1d_row_wgrad_kernel(const T* __restrict__ x,
                                                                         const T* __restrict__ g,
                                                                         float* __restrict__ partial, Row1D pl,
                                                                         int B, int per_chunk) {
  WT_SHARED_FLOATS(lds);
  constexpr int R = K / 2;
  constexpr int SLOT = row1d_slot(K, L, S);
  constexpr int NF = 1 + 2 * L;
  const int c = blockIdx.x;
  const int chunk = blockIdx.y;
  const int tid = threadIdx.x, nth = blockDim.x;
  constexpr int G = row1d_guard(K, L, S);
  float* xlds = lds + G * SLOT;                     // (regions point at the slot of lane 0, behind their left guard)
  float* glds = xlds + (nth + 2 * G) * SLOT;
  float* slot = xlds + tid * SLOT;
  const float* gslot = glds + tid * SLOT;
  row1d_zero_guards<K, L, S>(lds, 2, tid, nth);

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
  row1d_store_partial<K, NF>(acc, gsum, lds, partial + (static_cast<size_t>(chunk) * pl.C + c) * NRED, tid, nth);
}

constexpr int kRow1dBwdMaxLanes = 256;      // threads per workgroup of the fused backward kernel (register budget)
// (K, L) pairs the fused backward kernel is built for: its (1 + 2L) * K + 1 running sums per lane must leave room for
// the rest in 256 registers (beyond 50 sums, 45 with 32 samples per lane, the compiler spills; those pairs run the
// backward pass as two kernels).
constexpr bool row1d_bwd_built(int K, int L, int S) {
  return row1d_built(K, L, S) && (1 + 2 * L) * K <= (S == 16 ? 50 : 45);
}

// The whole backward pass of a row-resident shape in one kernel.  grid = (C, nchunk), block = lanes, dynamic LDS =
// 2 * block * SLOT floats (x slots, then grad_out slots, which also stage grad_x on its way out).  Per row: x and
// grad_out are read once; grad_x = the layer applied to grad_out with reversed taps and no bias; the correlation
// sums of x's pyramid with grad_out's go into (1 + 2L) * K + 1 running sums per lane.  After its rows a workgroup
// stores its record of sums and draws its channel's ticket; the last one of a channel runs the second stage
// (wgrad_finish_channel) for it and leaves the ticket zero.  `tickets`: C words, zero at launch.
template <typename T, int K, int L, int S>
__global__ __launch_bounds__(kRow1dBwdMaxLanes, 2) void wt1d_row_bwd_kernel(const T* __restrict__ x,
                                                                          const T* __restrict__ g,
                                                                          T* __restrict__ gx,
                                                                          float* __restrict__ partial,
                                                                          unsigned* __restrict__ tickets,
                                                                          const ParamTable prm, int pdtype,
                                                                          const GradTable gt, Row1D pl, int B,
                                                                          int per_chunk, int nchunk) {
  WT_SHARED_FLOATS(lds);
  constexpr int R = K / 2;
  constexpr int SLOT = row1d_slot(K, L, S);
  constexpr int NF = 1 + 2 * L;
  constexpr int EV = 16 / sizeof(T);
  const int c = blockIdx.x;
  const int chunk = blockIdx.y;
  const int tid = threadIdx.x, nth = blockDim.x;
  constexpr int G = row1d_guard(K, L, S);
  float* xlds = lds + G * SLOT;                     // (regions point at the slot of lane 0, behind their left guard)
  float* glds = xlds + (nth + 2 * G) * SLOT;
  float* xslot = xlds + tid * SLOT;
  float* gslot = glds + tid * SLOT;
  row1d_zero_guards<K, L, S>(lds, 2, tid, nth);
  const bool fast = pl.vec_ok != 0 && pl.N % EV == 0;

  RowWeights<K, L> fwc;
  row1d_fold<K, L>(prm, pdtype, c, 1, fwc);

  float acc[NF][K];
  float gsum = 0.f;
#pragma unroll
  for (int f = 0; f < NF; ++f)
#pragma unroll
    for (int k = 0; k < K; ++k) acc[f][k] = 0.f;

  const int b_end = (chunk + 1) * per_chunk < B ? (chunk + 1) * per_chunk : B;
  // with 16 samples per lane, rows on the fast path (16-byte sized and aligned) are fetched one row ahead into
  // registers; with 32 the registers for that are not there, and the rows are staged as the loop reaches them
  constexpr bool kAhead = S <= 16;
  const bool ahead = kAhead && fast;
  uint4 qx[kAhead ? S / EV : 1], qg[kAhead ? S / EV : 1];
  const int b_first = chunk * per_chunk;
  if (b_first < b_end && ahead) {
    const size_t r0 = (static_cast<size_t>(b_first) * pl.C + c) * pl.N;
    if constexpr (kAhead) {
      row1d_fetch<T, S, true>(x + r0, pl.N, tid, nth, qx);
      row1d_fetch<T, S, true>(g + r0, pl.N, tid, nth, qg);
      row1d_commit<T, S, SLOT>(xlds, pl.nl, tid, nth, qx);
      row1d_commit<T, S, SLOT>(glds, pl.nl, tid, nth, qg);
    }
  }
  for (int bv = b_first; bv < b_end; ++bv) {
    const int b = WT_UNIFORM(bv);
    const size_t roff = (static_cast<size_t>(b) * pl.C + c) * pl.N;
    const bool more = b + 1 < b_end;
    const size_t rnext = (static_cast<size_t>(more ? b + 1 : b) * pl.C + c) * pl.N;
    if (!ahead) {
      if (fast) {
        row1d_stage_pair<T, S, SLOT>(x + roff, g + roff, xlds, glds, pl.N, pl.nl, tid, nth);
      } else {
        row1d_stage_scalar<T, S, SLOT>(x + roff, xlds, pl.N, pl.nl, tid, nth);
        row1d_stage_scalar<T, S, SLOT>(g + roff, glds, pl.N, pl.nl, tid, nth);
      }
    }
    WT_LDS_BARRIER();
    float xs[S], gs[S];
    if (tid < pl.nl) {
      row1d_read_slot<S>(xslot, xs);
      row1d_read_slot<S>(gslot, gs);
    } else {
#pragma unroll
      for (int q = 0; q < S; ++q) { xs[q] = 0.f; gs[q] = 0.f; }
    }
    if constexpr (kAhead) {
      if (ahead && more) {
        row1d_fetch<T, S, true>(x + rnext, pl.N, tid, nth, qx);
        row1d_fetch<T, S, true>(g + rnext, pl.N, tid, nth, qg);
      }
    }
    row1d_publish<K, S, 0>(xslot, xs);
    row1d_publish<K, S, 0>(gslot, gs);
    row1d_publish_chain<K, S, L, 1>(xslot, xs);
    row1d_publish_chain<K, S, L, 1>(gslot, gs);
    WT_LDS_BARRIER();
    // (opaque from here on: otherwise the compiler keeps the coefficients it formed for the edges above alive across
    // the barrier instead of forming them again level by level)
    pin_values(xs);
    pin_values(gs);
    // base conv: its correlation sums, and its share of grad_x (the layer on grad_out with the reversed taps)
    float o[S];
#pragma unroll
    for (int e = 0; e < S; ++e) o[e] = 0.f;
    {
      float ext[S + 2 * R];
      row1d_extend<K, S, SLOT, 0>(xlds, tid, nth, xs, ext);
      row1d_corr<K, S>(ext, gs, acc[0]);
#pragma unroll
      for (int q = 0; q < S; ++q) gsum += gs[q];
    }
    {
      float ext[S + 2 * R];
      row1d_extend<K, S, SLOT, 0>(glds, tid, nth, gs, ext);
      row1d_conv<K, L, 0, S>(ext, fwc, o);
    }
    pin_values(o);
    WT_CHUNK_FENCE();
    row1d_bwd_levels<K, S, SLOT, L, 1>(xlds, glds, tid, nth, fwc, xs, gs, acc, o);
    WT_LDS_BARRIER();            // every neighbour has read this lane's edges
    row1d_write_slot<S>(gslot, o);
    WT_LDS_BARRIER();
    row1d_unstage<T, S, SLOT>(gx + roff, glds, pl.N, pl.vec_ok != 0, tid, nth);
    WT_LDS_BARRIER();            // the next row's staging overwrites the slots read above
    if constexpr (kAhead) {
      if (ahead && more) {
        row1d_commit<T, S, SLOT>(xlds, pl.nl, tid, nth, qx);
        row1d_commit<T, S, SLOT>(glds, pl.nl, tid, nth, qg);
      }
    }
  }

  constexpr int NRED = NF * K + 1;
  row1d_store_partial<K, NF, true>(acc, gsum, lds, partial + (static_cast<size_t>(chunk) * pl.C + c) * NRED, tid, nth);
  unsigned* flag = reinterpret_cast<unsigned*>(lds + (nth >> 6) * NRED);
  if (workgroup_is_last(tickets + c, static_cast<unsigned>(nchunk), flag)) {
    wgrad_finish_channel<true>(partial, nchunk, prm, pdtype, gt, pl.C, c, 2, L, K, lds);
    if (tid == 0) tickets[c] = 0u;
  }
}

}  // namespace wt
