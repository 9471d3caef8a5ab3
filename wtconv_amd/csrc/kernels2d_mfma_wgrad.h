// Parameter gradients of WTConv2d on the matrix cores of gfx950 (bf16 tensors, kernel size <= 5).
//
//   dW~_f[kh][kw] = sum over planes, i, j of  dY_f[i][j] * A_f[i + kh - 2][j + kw - 2]
// for every filter f of a channel (base conv: dY = grad_out, A = x; level l, sub-band s: the
// Haar pyramids of grad_out and of x; reference wtconv/wtconv2d.py:38-82 through autograd, and
// fast_wtconv/cuda_haar/haar_cuda.py:168-197 for the algebra).  Both pyramids of `pb` planes of
// one channel sit in LDS as bf16 images, the planes stacked with zero rows in between, so that
// one image per (level, sub-band) holds the whole unit.  The correlation runs as
// v_mfma_f32_16x16x32_bf16 with the contraction along image rows:
//     D_kw[m][n] += sum_j A[R0 - 2 + m][j] * dY[R0 + n][j - kw + 2]
// (M = 16 rows of A, N = 16 rows of dY, K = 32 columns); tap (kh, kw) is the sum of the
// diagonal m - n = kh over n < 12, so a row tile advances by 12 rows and five accumulators
// (one per kw) serve a filter.  The column shift by kw - 2 is made in registers: a lane loads
// 12 consecutive bf16 of a dY row and funnel-shifts the odd offsets.  Accumulators stay in
// registers over the whole batch chunk of the workgroup; wave w owns sub-band w % 4 of every
// level (with eight waves, every second row tile of it) and its share of the base-conv tiles.
// Partial sums go to the workspace in the layout wgrad_finish_kernel (kernels2d.h) reduces,
// deterministically.
//
// Precision: the pixels are bf16 already, so the base-conv products are exact.  Haar coefficients
// need more than 8 mantissa bits; rounding both pyramids to bf16 leaves a relative error of about
// 0.16 % per product, whose tail reaches the 2e-2 bar on the rare tap dominated by a few large
// products.  The coefficients of x are therefore kept as two bf16 planes (hi + lo, 16 bits) and
// both products are accumulated, which leaves the rounding of the grad_out coefficients only.
// Levels up to 16 columns wide put hi and lo side by side in the contraction (16 columns x 2
// planes = 32) against the dY window taken twice: one MFMA per kw instead of two.
#pragma once

#include "common.h"
#include "kernels2d_mfma.h"
#include "wgrad_finish.h"

namespace wt {

constexpr int kWgRowStep = 12;       // dY rows per tile whose five kernel rows fit the 16 rows of A

struct WPlan {
  int B, C, H, W, L;
  int pb;                            // planes per unit (stacked images)
  int h[kMaxLevels + 1], w[kMaxLevels + 1];
  int nbr[kMaxLevels + 1], nbc[kMaxLevels + 1], bpp0, nblk0;
  unsigned mg_bpp0, mg_nbc0;
  unsigned mg_hw[kMaxLevels + 1], mg_w[kMaxLevels + 1];
  int prows[kMaxLevels + 1];         // image rows from one stacked plane to the next: 4 nbr + 2
  // dY images: zero halo of 2 (element (p, r, c) at row p*prows + r + 2, column c + 2)
  int gpitch[kMaxLevels + 1], goff[kMaxLevels + 1], gsub[kMaxLevels + 1];
  // A images: rows as above, columns unshifted (element column c); from level 1 on a second (lo) plane
  // per sub-band follows the four hi planes
  int xpitch[kMaxLevels + 1], xoff[kMaxLevels + 1], xsub[kMaxLevels + 1];
  // The 32-long contraction of an MFMA covers kc = 32, 16 or 8 columns; what is left of it holds the second
  // split plane of A (levels >= 1) and then `fold` row tiles at once.
  int kc[kMaxLevels + 1], fold[kMaxLevels + 1];
  int nrt[kMaxLevels + 1], nct[kMaxLevels + 1];    // row tiles (of 12 rows), column tiles (kc = 32 only)
  int llxoff[kMaxLevels + 1], llgoff[kMaxLevels + 1], llpl[kMaxLevels + 1];   // fp32 raw LL, 2 <= l < L
  int zero_off;
  int lds_bytes;
};

// Shape-dependent part of the plan (constexpr: compile-time constant for the common shapes).
// `compact` gives the narrow levels from 2 on rows of an even number of 16-byte units (two-way bank conflicts
// on their loads) where that brings a single plane under the LDS of two workgroups per CU.
constexpr bool make_wplan_geometry(int H, int W, int L, int pb, int nthreads, bool compact, WPlan* out) {
  auto cdiv = [](int a, int b) { return (a + b - 1) / b; };
  auto rup = [](int v, int m) { return (v + m - 1) / m * m; };
  auto odd8 = [](int v) { v = (v + 7) / 8 * 8; return (v / 8) % 2 == 0 ? v + 8 : v; };   // rows of an odd number of 16-byte units: 16 consecutive rows fall into distinct banks
  WPlan pl = {};
  pl.H = H; pl.W = W; pl.L = L;
  pl.pb = pb;
  pl.h[0] = H; pl.w[0] = W;
  for (int l = 1; l <= L; ++l) { pl.h[l] = (pl.h[l - 1] + 1) / 2; pl.w[l] = (pl.w[l - 1] + 1) / 2; }
  int off = 0;
  for (int l = 0; l <= L; ++l) {
    pl.nbr[l] = cdiv(pl.h[l], 4);
    pl.nbc[l] = cdiv(pl.w[l], 4);
    pl.prows[l] = 4 * pl.nbr[l] + 2;
    pl.nrt[l] = cdiv(pb * pl.prows[l], kWgRowStep);
    pl.kc[l] = pl.w[l] > 16 ? 32 : pl.w[l] > 8 ? 16 : 8;
    pl.nct[l] = pl.kc[l] == 32 ? cdiv(pl.w[l], 32) : 1;
    pl.fold[l] = l == 0 ? 32 / pl.kc[l] : (pl.kc[l] == 32 ? 1 : 16 / pl.kc[l]);
    // the last tile reads rows past the stacked planes; a level of fewer row tiles than lane groups parks the
    // groups left over on a block of zeros instead
    const int rows = kWgRowStep * (pl.nrt[l] < pl.fold[l] ? pl.nrt[l] : rup(pl.nrt[l], pl.fold[l])) + 6;
    const bool cmp = compact && l >= 2 && pl.kc[l] <= 16;
    pl.gpitch[l] = cmp ? rup(4 * pl.nbc[l] + 4, 8) : odd8(4 * pl.nbc[l] + 4);
    pl.xpitch[l] = pl.kc[l] == 32 ? odd8(32 * pl.nct[l]) : pl.kc[l] == 16 ? (cmp ? 16 : 24) : 8;
    if (l >= 3) {
      if (!make_magic(pl.h[l] * pl.w[l], 2 * pb * pl.h[l] * pl.w[l] + nthreads, &pl.mg_hw[l])) return false;
      if (!make_magic(pl.w[l], pl.h[l] * pl.w[l], &pl.mg_w[l])) return false;
    }
    pl.goff[l] = off;
    pl.gsub[l] = rup(rows * pl.gpitch[l] * 2, 16);
    off += pl.gsub[l] * (l == 0 ? 1 : 4);
    pl.xoff[l] = off;
    pl.xsub[l] = rup(rows * pl.xpitch[l] * 2, 16);
    off += pl.xsub[l] * (l == 0 ? 1 : 8);
    if (off > (1 << 20)) return false;
  }
  pl.bpp0 = pl.nbr[0] * pl.nbc[0];
  pl.nblk0 = pb * pl.bpp0;
  if (pl.nblk0 > kMfmaBlock) return false;              // one 4x4 block per thread of four waves
  if (!make_magic(pl.bpp0, kMfmaBlock, &pl.mg_bpp0)) return false;
  if (!make_magic(pl.nbc[0], pl.bpp0, &pl.mg_nbc0)) return false;
  for (int l = 2; l < L; ++l) {
    pl.llpl[l] = pl.h[l] * pl.w[l];
    pl.llxoff[l] = off;
    off += rup(pb * pl.llpl[l] * 4, 16);
    pl.llgoff[l] = off;
    off += rup(pb * pl.llpl[l] * 4, 16);
  }
  pl.zero_off = off;   // 64 bytes that stay zero: a dY window may end a few elements past its image, idle lane groups read A here
  off += 64;
  // the final reduction reuses the images: per wave the five diagonals of 12 elements of 5 (1 + L) tiles
  if (off < 8 * ((1 + L) * 5 * 5 * kWgRowStep * 4 + 4)) off = 8 * ((1 + L) * 5 * 5 * kWgRowStep * 4 + 4);
  pl.lds_bytes = rup(off, 16);
  *out = pl;
  return true;
}

struct WGeoRuntime {
  static constexpr bool kStatic = false;
};
template <int H, int W, int L, int PB, int NT, bool COMPACT>
struct WGeoStatic {
  static constexpr bool kStatic = true;
  static constexpr WPlan plan() {
    WPlan p = {};
    make_wplan_geometry(H, W, L, PB, NT, COMPACT, &p);
    return p;
  }
};

// Which taps of the 5 x 5 frame a kernel size uses: K = 5 all, K = 3 the centre 3 x 3, K = 1 the centre.
__device__ __forceinline__ int tap_of_frame(int kh, int kw, int K) {
  const int o = 2 - K / 2;
  const int ih = kh - o, iw = kw - o;
  return (ih >= 0 && ih < K && iw >= 0 && iw < K) ? ih * K + iw : -1;
}

// Operands of one tile: rows R0-2.. of an A image (NX split planes) against rows R0.. of a dY image.
template <int NX>
struct CorrTile {
  Frag a[NX];        // A rows: 8 bf16 at an aligned column
  uint32_t w[6];     // dY rows: 12 bf16 from the aligned column index of the tile (the halo of 2 makes that element - 2)
};

template <int NX>
__device__ __forceinline__ void corr_load(const char* lds, int xbase, int xsplit, int gbase, CorrTile<NX>& t) {
#pragma unroll
  for (int i = 0; i < NX; ++i) t.a[i] = lds_frag16(lds, xbase + i * xsplit);
  const uint4 w03 = lds_ld<uint4>(lds, gbase);
  const uint2 w45 = lds_ld<uint2>(lds, gbase + 16);
  t.w[0] = w03.x; t.w[1] = w03.y; t.w[2] = w03.z; t.w[3] = w03.w; t.w[4] = w45.x; t.w[5] = w45.y;
}

template <int NX>
__device__ __forceinline__ void corr_mma(const CorrTile<NX>& t, Acc (&d)[5]) {
  const uint32_t* w = t.w;
  uint32_t s[5];                     // s[i] = elements (2i + 1, 2i + 2)
#ifdef WT_EMULATE
#pragma unroll
  for (int i = 0; i < 5; ++i) s[i] = (w[i] >> 16) | (w[i + 1] << 16);
#else
#pragma unroll
  for (int i = 0; i < 5; ++i) s[i] = __builtin_amdgcn_alignbit(w[i + 1], w[i], 16);
#endif
  // kw -> first element 4 - kw of the window
  Frag b[5];
  b[0].d[0] = w[2]; b[0].d[1] = w[3]; b[0].d[2] = w[4]; b[0].d[3] = w[5];
  b[1].d[0] = s[1]; b[1].d[1] = s[2]; b[1].d[2] = s[3]; b[1].d[3] = s[4];
  b[2].d[0] = w[1]; b[2].d[1] = w[2]; b[2].d[2] = w[3]; b[2].d[3] = w[4];
  b[3].d[0] = s[0]; b[3].d[1] = s[1]; b[3].d[2] = s[2]; b[3].d[3] = s[3];
  b[4].d[0] = w[0]; b[4].d[1] = w[1]; b[4].d[2] = w[2]; b[4].d[3] = w[3];
#pragma unroll
  for (int jx = NX - 1; jx >= 0; --jx)      // the small (lo) plane first
#pragma unroll
    for (int kw = 0; kw < 5; ++kw) mfma_bf16(t.a[jx], b[kw], d[kw]);
}

// Grid (C, nchunk): workgroup (c, k) sums over batch items [k * bchunk, (k + 1) * bchunk) of channel c.
// NW = 4 or 8 waves per workgroup.
template <int L, int NW, bool VEC, typename Geo>
__global__ void __launch_bounds__(NW * 64, 2)
wt2d_mfma_wgrad_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ g, float* __restrict__ partial,
                       const WPlan plarg, int K, int bchunk, const FinishArgs fin) {
  const WPlan pl = [&]() {
    if constexpr (Geo::kStatic) {
      constexpr WPlan gp = Geo::plan();
      WPlan p = gp;
      p.B = plarg.B; p.C = plarg.C;
      return p;
    } else {
      return plarg;
    }
  }();
  constexpr int NT = NW * 64, NH = NW / 4;
  WT_SHARED_FLOATS(ldsf);
  char* lds = reinterpret_cast<char*>(ldsf);
  const int tid = threadIdx.x, lane = tid & 63, wave = WT_UNIFORM(tid >> 6);
  const int sb = wave & 3, half = wave >> 2;
  const int n = lane & 15, q = lane >> 4;
  const int H = pl.H, W = pl.W, HW = H * W, C = pl.C, B = pl.B, pb = pl.pb;
  const int c = xcd_contiguous(blockIdx.x, gridDim.x);
  const int b_begin = blockIdx.y * bchunk;
  const int b_end = b_begin + bchunk < B ? b_begin + bchunk : B;

  // ---- commit role: one 4x4 pixel block per thread of four waves -- of x and of grad_out, or with eight
  // waves of x in the first four and of grad_out in the others
  constexpr bool kSplitCommit = NW == 8;
  const int ctid = tid & 255;
  const bool act = ctid < pl.nblk0 && (kSplitCommit || tid < 256);
  const int gg = act ? ctid : 0;
  const int cp = fast_div(gg, pl.mg_bpp0);
  const int rem = gg - imul(cp, pl.bpp0);
  const int bi = fast_div(rem, pl.mg_nbc0);
  const int bj = rem - imul(bi, pl.nbc[0]);
  unsigned cmask = act ? 0x100u : 0u;
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    if (4 * bi + r < H) cmask |= 1u << r;
    if (4 * bj + r < W) cmask |= 16u << r;
  }
  const int c_goff = cp * C * HW + 4 * bi * W + 4 * bj;
  const int row0 = cp * pl.prows[0] + 4 * bi + 2, row1 = cp * pl.prows[1] + 2 * bi + 2;
  const int row2 = L >= 2 ? cp * pl.prows[L >= 2 ? 2 : 0] + bi + 2 : 0;
  const int x_l0 = pl.xoff[0] + (row0 * pl.xpitch[0] + 4 * bj) * 2;
  const int g_l0 = pl.goff[0] + (row0 * pl.gpitch[0] + 4 * bj + 2) * 2;
  const int x_l1 = pl.xoff[1] + (row1 * pl.xpitch[1] + 2 * bj) * 2;
  const int g_l1 = pl.goff[1] + (row1 * pl.gpitch[1] + 2 * bj + 2) * 2;
  const int x_l2 = L >= 2 ? pl.xoff[L >= 2 ? 2 : 0] + (row2 * pl.xpitch[L >= 2 ? 2 : 0] + bj) * 2 : 0;
  const int g_l2 = L >= 2 ? pl.goff[L >= 2 ? 2 : 0] + (row2 * pl.gpitch[L >= 2 ? 2 : 0] + bj + 2) * 2 : 0;
  const int ll_i = L >= 3 ? (cp * pl.llpl[L >= 3 ? 2 : 0] + bi * pl.w[L >= 3 ? 2 : 0] + bj) * 4 : 0;
  const int xsub2 = pl.xsub[L >= 2 ? 2 : 0], gsub2 = pl.gsub[L >= 2 ? 2 : 0];
  const int llx2 = pl.llxoff[L >= 3 ? 2 : 0], llg2 = pl.llgoff[L >= 3 ? 2 : 0];

  using Pix = PixRow<bf16_t>;
  Pix px[4], pg[kSplitCommit ? 1 : 4];
  const bf16_t* src0 = (kSplitCommit && half) ? g : x;
  const size_t total_elems = static_cast<size_t>(B) * C * HW;
  const uint2 colmask = pix_col_mask(cmask);
  auto fetch = [&](int b0) {
    const size_t base = (static_cast<size_t>(b0) * C + c) * HW;
    const bool plane_ok = act && b0 + cp < b_end;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      pix_zero(px[r]);
      if constexpr (!kSplitCommit) pix_zero(pg[r]);
      if (plane_ok && (cmask >> r & 1u)) {
        const bf16_t* sx = src0 + base + c_goff + r * W;
        const bf16_t* sg = g + base + c_goff + r * W;
        if constexpr (VEC) {
          if (cmask & 16u) {
            pix_load4(px[r], sx);
            if constexpr (!kSplitCommit) pix_load4(pg[r], sg);
          }
        } else if (base + c_goff + r * W + 4 <= total_elems) {
          // rows that are not whole aligned vectors: still one (unaligned) 8-byte load per row; the columns that
          // come along from past the row end are cleared at the commit
          pix_load4u(px[r].v, sx);
          if constexpr (!kSplitCommit) pix_load4u(pg[r].v, sg);
        } else {      // the four elements would reach past the end of the tensor: element by element
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (cmask >> (4 + e) & 1u) {
              pix_set(px[r], e, sx[e]);
              if constexpr (!kSplitCommit) pix_set(pg[r], e, sg[e]);
            }
        }
      }
    }
  };
  if (b_begin < b_end) fetch(b_begin);

  // halos, padding rows and the rows of planes past the batch stay zero from here on
  for (int o = tid * 16; o < pl.lds_bytes; o += NT * 16) {
    uint4 z; z.x = z.y = z.z = z.w = 0u;
    lds_st<uint4>(lds, o, z);
  }
  WT_LDS_BARRIER();

  // pixels -> level-0 image; levels 1 and 2 from registers (N1 split planes each); the raw LL of level 2 to `llo`
  auto commit = [&](const Pix (&pr)[4], int o0, int pitch0, bool pair64, int o1, int pitch1, int sub1, int o2,
                    int sub2, int llo, float& llsum, auto n1) {
    constexpr int N1 = decltype(n1)::value;
    float v[4][4];
    Pix row[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      row[r] = pr[r];
      if constexpr (!VEC) { row[r].v.x &= colmask.x; row[r].v.y &= colmask.y; }
      pix_get(row[r], v[r]);
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const uint2 w = pix_words(row[r]);
      if (pair64) {
        lds_st<uint2>(lds, o0 + r * pitch0 * 2, w);
      } else {
        lds_st<uint32_t>(lds, o0 + r * pitch0 * 2, w.x);
        lds_st<uint32_t>(lds, o0 + r * pitch0 * 2 + 4, w.y);
      }
    }
    float ll1[2][2];
#pragma unroll
    for (int i2 = 0; i2 < 2; ++i2) {
      float cf[4][2];
#pragma unroll
      for (int j2 = 0; j2 < 2; ++j2) {
        const float a = v[2 * i2][2 * j2], b = v[2 * i2][2 * j2 + 1];
        const float cc = v[2 * i2 + 1][2 * j2], d = v[2 * i2 + 1][2 * j2 + 1];
        const float s1 = a + b, d1 = a - b, s2 = cc + d, d2 = cc - d;
        cf[0][j2] = s1 + s2; cf[1][j2] = s1 - s2; cf[2][j2] = d1 + d2; cf[3][j2] = d1 - d2;
      }
      ll1[i2][0] = cf[0][0]; ll1[i2][1] = cf[0][1];
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        uint32_t wv[N1];
        split_pair<N1>(cf[s][0], cf[s][1], wv);
#pragma unroll
        for (int j = 0; j < N1; ++j) lds_st<uint32_t>(lds, o1 + (j * 4 + s) * sub1 + i2 * pitch1 * 2, wv[j]);
      }
    }
    if (L == 1) llsum += (ll1[0][0] + ll1[0][1]) + (ll1[1][0] + ll1[1][1]);
    if (L >= 2) {
      const float a = ll1[0][0], b = ll1[0][1], cc = ll1[1][0], d = ll1[1][1];
      const float s1 = a + b, d1 = a - b, s2 = cc + d, d2 = cc - d;
      const float cf[4] = {s1 + s2, s1 - s2, d1 + d2, d1 - d2};
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        uint32_t wv[N1];
        split_pair<N1>(cf[s], 0.f, wv);
#pragma unroll
        for (int j = 0; j < N1; ++j) lds_st<uint16_t>(lds, o2 + (j * 4 + s) * sub2, static_cast<uint16_t>(wv[j]));
      }
      if (L == 2) llsum += cf[0];
      if (L >= 3) lds_st<float>(lds, llo, cf[0]);
    }
  };

  Acc db[5], dl[L][5];
#pragma unroll
  for (int k = 0; k < 5; ++k) {
    db[k].v[0] = db[k].v[1] = db[k].v[2] = db[k].v[3] = 0.f;
#pragma unroll
    for (int l = 0; l < L; ++l) dl[l][k].v[0] = dl[l][k].v[1] = dl[l][k].v[2] = dl[l][k].v[3] = 0.f;
  }
  float gsum = 0.f, no_sum = 0.f;      // (the LL sum of x is not needed)

  // one level of both pyramids from the raw LL of the level above (fp32 in LDS)
  auto analyse = [&](auto lc) {
    const int l = lc;
    const int hl = pl.h[l], wl = pl.w[l], npos = pb * hl * wl;
    for (int idx = tid; idx < 2 * npos; idx += NT) {
      const bool is_g = idx >= npos;
      const int id = is_g ? idx - npos : idx;
      const int p = fast_div(id, pl.mg_hw[l]);
      const int rm = id - imul(p, hl * wl);
      const int i = fast_div(rm, pl.mg_w[l]);
      const int j = rm - imul(i, wl);
      const int hs = pl.h[l - 1], wsrc = pl.w[l - 1];
      const int so = (is_g ? pl.llgoff[l - 1] : pl.llxoff[l - 1]) + (imul(p, pl.llpl[l - 1]) + imul(2 * i, wsrc) + 2 * j) * 4;
      const bool r1 = 2 * i + 1 < hs, c1 = 2 * j + 1 < wsrc;
      const float a = lds_ld<float>(lds, so);
      const float b = c1 ? lds_ld<float>(lds, so + 4) : 0.f;
      const float cc = r1 ? lds_ld<float>(lds, so + wsrc * 4) : 0.f;
      const float d = (r1 && c1) ? lds_ld<float>(lds, so + wsrc * 4 + 4) : 0.f;
      const float s1 = a + b, d1 = a - b, s2 = cc + d, d2 = cc - d;
      const float cf[4] = {s1 + s2, s1 - s2, d1 + d2, d1 - d2};
      const int row = imul(p, pl.prows[l]) + i + 2;
      const int ao = is_g ? pl.goff[l] + (imul(row, pl.gpitch[l]) + j + 2) * 2 : pl.xoff[l] + (imul(row, pl.xpitch[l]) + j) * 2;
      const int sub = is_g ? pl.gsub[l] : pl.xsub[l];
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        uint32_t wv[2];
        split_pair<2>(cf[s], 0.f, wv);
        lds_st<uint16_t>(lds, ao + s * sub, static_cast<uint16_t>(wv[0]));
        if (!is_g) lds_st<uint16_t>(lds, ao + (4 + s) * sub, static_cast<uint16_t>(wv[1]));
      }
      if (l < L) lds_st<float>(lds, (is_g ? pl.llgoff[l] : pl.llxoff[l]) + (imul(p, pl.llpl[l]) + imul(i, wl) + j) * 4, cf[0]);
      else if (is_g) gsum += cf[0];
    }
    WT_LDS_BARRIER();
  };

  // A lane's share of the contraction at level l: its group q of eight k-values is a column group, and where
  // columns leave room the second split plane of A and further row tiles.
  auto lane_x = [&](int l, int sub) {
    const int kc = pl.kc[l];
    const int cg = kc == 32 ? q : kc == 16 ? (q & 1) : 0;
    const int g2 = kc == 32 ? 0 : kc == 16 ? (q >> 1) : q;
    const int split = l == 0 ? 0 : (g2 & 1), toff = l == 0 ? g2 : (g2 >> 1);
    if (toff >= pl.nrt[l]) return pl.zero_off;      // no such row tile: zeros
    return pl.xoff[l] + (split * 4 + sub) * pl.xsub[l] + imul(n + kWgRowStep * toff, pl.xpitch[l] * 2) + 16 * cg;
  };
  auto lane_g = [&](int l) {
    const int kc = pl.kc[l];
    const int cg = kc == 32 ? q : kc == 16 ? (q & 1) : 0;
    const int g2 = kc == 32 ? 0 : kc == 16 ? (q >> 1) : q;
    const int toff0 = l == 0 ? g2 : (g2 >> 1);
    const int toff = toff0 >= pl.nrt[l] ? 0 : toff0;
    return pl.goff[l] + imul(2 + n + kWgRowStep * toff, pl.gpitch[l] * 2) + 16 * cg;
  };

  // correlations of sub-band `sb` of one level: this wave's row tiles
  auto level_pass = [&](auto lc) {
    constexpr int l = decltype(lc)::value;
    const int xp = pl.xpitch[l] * 2, gp = pl.gpitch[l] * 2, nct = pl.nct[l], nrt = pl.nrt[l], fold = pl.fold[l];
    const int xo = lane_x(l, sb), go = lane_g(l) + sb * pl.gsub[l];
    if (pl.kc[l] == 32) {        // wide level: the two split planes of A take an MFMA each
      const int xsplit = 4 * pl.xsub[l];
#pragma unroll 1
      for (int rt = half; rt < nrt; rt += NH)
#pragma unroll 2
        for (int ct = 0; ct < nct; ++ct) {
          CorrTile<2> t;
          corr_load<2>(lds, xo + rt * kWgRowStep * xp + 64 * ct, xsplit, go + rt * kWgRowStep * gp + 64 * ct, t);
          corr_mma<2>(t, dl[l - 1]);
        }
    } else {
#pragma unroll 2
      for (int rt = half * fold; rt < nrt; rt += NH * fold) {
        CorrTile<1> t;
        corr_load<1>(lds, xo + rt * kWgRowStep * xp, 0, go + rt * kWgRowStep * gp, t);
        corr_mma<1>(t, dl[l - 1]);
      }
    }
  };

#pragma unroll 1
  for (int b0 = b_begin; b0 < b_end; b0 += pb) {
    if (act) {
      using std::integral_constant;
      if (!kSplitCommit || half == 0)
        commit(px, x_l0, pl.xpitch[0], true, x_l1, pl.xpitch[1], pl.xsub[1], x_l2, xsub2, llx2 + ll_i, no_sum,
               integral_constant<int, 2>{});
      if constexpr (kSplitCommit) {
        if (half == 1)
          commit(px, g_l0, pl.gpitch[0], false, g_l1, pl.gpitch[1], pl.gsub[1], g_l2, gsub2, llg2 + ll_i, gsum,
                 integral_constant<int, 1>{});
      } else {
        commit(pg, g_l0, pl.gpitch[0], false, g_l1, pl.gpitch[1], pl.gsub[1], g_l2, gsub2, llg2 + ll_i, gsum,
               integral_constant<int, 1>{});
      }
    }
    if (b0 + pb < b_end) fetch(b0 + pb);
    WT_LDS_BARRIER();
    {
      using std::integral_constant;
      if constexpr (L >= 3) analyse(integral_constant<int, 3>{});
      if constexpr (L >= 4) analyse(integral_constant<int, 4>{});
      if constexpr (L >= 5) analyse(integral_constant<int, 5>{});
    }
    // ---- correlations: base-conv tiles round-robin over the waves, then this wave's sub-band of every level
    {
      const int nct0 = pl.nct[0], fold = pl.fold[0], ntile = (pl.nrt[0] + fold - 1) / fold * nct0;
      const int xp = pl.xpitch[0] * 2 * fold, gp = pl.gpitch[0] * 2 * fold;
      const int xo = lane_x(0, 0), go = lane_g(0);
#pragma unroll 2
      for (int t = wave; t < ntile; t += NW) {
        const int rt = nct0 == 1 ? t : (t >> 1), cc = nct0 == 1 ? 0 : (t & 1);       // planes up to 64 wide: one or two column tiles
        CorrTile<1> ct;
        corr_load<1>(lds, xo + rt * kWgRowStep * xp + 64 * cc, 0, go + rt * kWgRowStep * gp + 64 * cc, ct);
        corr_mma<1>(ct, db);
      }
    }
    {
      using std::integral_constant;
      level_pass(integral_constant<int, 1>{});
      if constexpr (L >= 2) level_pass(integral_constant<int, 2>{});
      if constexpr (L >= 3) level_pass(integral_constant<int, 3>{});
      if constexpr (L >= 4) level_pass(integral_constant<int, 4>{});
      if constexpr (L >= 5) level_pass(integral_constant<int, 5>{});
    }
    WT_LDS_BARRIER();
  }

  // ---- taps: tap (kh, kw) of a filter = sum over n < 12 of D_kw[n + kh][n]; lane (n, q) holds D[4q + r][n].
  // Every wave leaves the five diagonals of its tiles in LDS (the images are dead after the last barrier),
  // then the threads sum them: over n, and over the waves that shared a filter.
  const int KK = K * K;
  const int nrec = (1 + 4 * L) * KK + 1;
  float* rec = partial + (static_cast<size_t>(blockIdx.y) * C + c) * nrec;
  constexpr int kBand = 5 * kWgRowStep * 4;                 // bytes of the diagonals of one tile
  constexpr int kWaveBand = (1 + L) * 5 * kBand;            // ... of one wave: tiles [filter][kw]
  auto put = [&](const Acc& d, int slot) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int kh = 4 * q + r - n;
      if (kh >= 0 && kh < 5 && n < kWgRowStep) lds_st<float>(lds, wave * kWaveBand + slot * kBand + (kh * kWgRowStep + n) * 4, d.v[r]);
    }
  };
#pragma unroll
  for (int kw = 0; kw < 5; ++kw) {
    put(db[kw], kw);
#pragma unroll
    for (int l = 1; l <= L; ++l) put(dl[l - 1][kw], l * 5 + kw);
  }
  const float gs = wave_sum(gsum);
  if (lane == 0) lds_st<float>(lds, NW * kWaveBand + wave * 4, gs);
  WT_LDS_BARRIER();
  for (int i = tid; i < 25 * (1 + 4 * L) + 1; i += NT) {
    float v = 0.f;
    if (i == 25 * (1 + 4 * L)) {
#pragma unroll
      for (int wv = 0; wv < NW; ++wv) v += lds_ld<float>(lds, NW * kWaveBand + wv * 4);
      if (fin.tickets != nullptr) store_shared_f32(rec + nrec - 1, v);
      else rec[nrec - 1] = v;
      continue;
    }
    const int f = i / 25, tap = i - 25 * f;          // f = 0: base conv; else 1 + 4 (l - 1) + s
    const int kh = tap / 5, kw = tap - 5 * kh;
    const int l = f == 0 ? 0 : ((f - 1) >> 2) + 1;
    const int w0 = f == 0 ? 0 : ((f - 1) & 3), wstep = f == 0 ? 1 : 4;      // base conv: every wave; sub-band s: waves s, s + 4, ...
    const int o = (l * 5 + kw) * kBand + kh * kWgRowStep * 4;
    for (int wv = w0; wv < NW; wv += wstep) {
      float4 t[3];
#pragma unroll
      for (int j = 0; j < 3; ++j) t[j] = lds_ld<float4>(lds, wv * kWaveBand + o + 16 * j);
      v += ((t[0].x + t[0].y) + (t[0].z + t[0].w)) + ((t[1].x + t[1].y) + (t[1].z + t[1].w)) +
           ((t[2].x + t[2].y) + (t[2].z + t[2].w));
    }
    float sc = 1.f;
    for (int k = 0; k < l; ++k) sc *= 0.25f;        // both pyramids were left unnormalised: 2^l each
    const int t = tap_of_frame(kh, kw, K);
    if (t >= 0) {
      if (fin.tickets != nullptr) store_shared_f32(rec + f * KK + t, v * sc);
      else rec[f * KK + t] = v * sc;
    }
  }
  wgrad_finish_if_last(fin, partial, static_cast<int>(gridDim.y), C, c, 4, L, KK, reinterpret_cast<float*>(lds));
}

}  // namespace wt
